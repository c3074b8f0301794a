// KVStar multi-query softmax-vote retrieval.
//
// Per task (one request in one layer): x <= 8 query tokens x H query heads are
// scored against every sub-block representative of the request,
//     score[x][H][s] = q[x][H] . k[s][h(H)],      s = block*M + sub-block,
// each (x, H) row is soft-maxed over s, and a block's vote is the sum of its
// sub-blocks' probabilities over all rows; the top-k blocks by vote are kept
// (ucm/sparse/kvstar/retrieve/core/domain/retrieve_task/simd_compute_kernel.cpp:817-990).
//
// Unlike single-query scoring this is a real contraction: the x*g rows that
// share a kv head reuse every representative, 2*x*g flop per 2 bytes (32-64
// flop/B), more than the vector ALUs can deliver at HBM speed, so it runs on the
// matrix cores (v_mfma_f32_32x32x16_f16) - and it still streams the table once.
// The product is taken with the representatives as the A operand and the
// queries as B, which leaves a lane with ONE query row and sixteen of a tile's
// 32 sub-blocks in registers: the row's maximum and the per-block sums of
// exp(score - max) are in-register work plus one exchange between the two lane
// halves.  Every 32-sub-block tile emits its row maxima and per-block partial
// sums (1/M of the score matrix); a second kernel rescales them to the global
// row maximum, normalises and adds the rows up.  fp32 throughout; the summation
// order differs from the reference's scalar loop, so results agree with it to
// rounding (a few 1e-6 relative), not bit for bit.
#include <algorithm>
#include <cmath>

#include "common.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
using ucm::u32x4;

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kMaxRows = 64;          // tokens * group size per kv head
constexpr int kMaxDim = 128;
constexpr int kQStride = kMaxDim + 8; // fp16 elements per staged query row (272 B: spreads LDS banks)
constexpr int kTileSub = 32;          // sub-blocks per MFMA tile

__device__ __forceinline__ unsigned short f32_to_f16_bits(float f)
{
    const _Float16 h = static_cast<_Float16>(f);
    return __builtin_bit_cast(unsigned short, h);
}

// ---- sub-block representatives -------------------------------------------------------------
// Table layout, per kv head: [row (block slot)][piece = d_pad/8][sub-block m][8 channels], fp16.  A
// block's representatives are one contiguous M*d_pad*2 bytes; inside it the 16-byte pieces of the M
// sub-blocks that an MFMA step multiplies together are adjacent, so one load instruction of the
// score kernel reads whole 128-byte lines (M*16 bytes per piece and block) instead of 16 bytes out
// of each of 64 lines.
//
// grid: x = listed block, y = layer.  Phase 1: a thread owns 8 adjacent columns of a token row
// (one 16-byte load per token, `merge` tokens accumulated in token order in fp32), the means -
// rounded to bf16 and then fp16, what mean() in the model dtype followed by .to(float16) gives -
// are parked in LDS as [M][kv_heads*head_dim].  Phase 2 gathers the kept channels from LDS and
// writes the block's pieces, consecutive threads to consecutive 16 bytes.
constexpr int kRepreUnroll = 16;

__device__ __forceinline__ unsigned mean_to_f16x2(float lo, float hi, float inv)
{
    unsigned a = __float_as_uint(lo * inv), b = __float_as_uint(hi * inv);
    a += 0x7fffu + ((a >> 16) & 1u);
    b += 0x7fffu + ((b >> 16) & 1u);
    return static_cast<unsigned>(f32_to_f16_bits(__uint_as_float(a & 0xffff0000u))) |
           (static_cast<unsigned>(f32_to_f16_bits(__uint_as_float(b & 0xffff0000u))) << 16);
}

__device__ __forceinline__ void add_bf16x8(float (&acc)[8], const u32x4 v)
{
    acc[0] = acc[0] + __uint_as_float(v.x << 16); acc[1] = acc[1] + __uint_as_float(v.x & 0xffff0000u);
    acc[2] = acc[2] + __uint_as_float(v.y << 16); acc[3] = acc[3] + __uint_as_float(v.y & 0xffff0000u);
    acc[4] = acc[4] + __uint_as_float(v.z << 16); acc[5] = acc[5] + __uint_as_float(v.z & 0xffff0000u);
    acc[6] = acc[6] + __uint_as_float(v.w << 16); acc[7] = acc[7] + __uint_as_float(v.w & 0xffff0000u);
}

__global__ __launch_bounds__(kThreads) void kvstar_repre_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned rows, unsigned block_size, unsigned kv_heads,
    unsigned head_dim, unsigned merge, const int32_t* __restrict__ pruned, unsigned d_pruned, unsigned d_pad,
    unsigned short* __restrict__ repre, int64_t layer_stride, int64_t head_stride)
{
    extern __shared__ __attribute__((aligned(16))) unsigned short stage[];   // [M][row]
    const unsigned M = block_size / merge;
    const unsigned id = static_cast<unsigned>(block_ids[blockIdx.x]);
    const unsigned slot = static_cast<unsigned>(slots[blockIdx.x]);
    if (id >= num_blocks || slot >= rows) { return; }   // whole workgroup: never dereference a bad id
    const unsigned row = kv_heads * head_dim, ncg = row / 8;
    const unsigned short* blk = static_cast<const unsigned short*>(k_layers[blockIdx.y]) +
                                static_cast<size_t>(id) * block_size * row;
    const float inv = 1.0f / static_cast<float>(merge);
    for (unsigned w = threadIdx.x; w < M * ncg; w += kThreads) {
        const unsigned m = w / ncg, cg = w - m * ncg;
        const unsigned short* src = blk + static_cast<size_t>(m) * merge * row + cg * 8;
        float acc[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) { acc[c] = -0.0f; }   // -0 + x == x for every x, signed zeros included
        unsigned t = 0;
        for (; t + kRepreUnroll <= merge; t += kRepreUnroll) {
            u32x4 v[kRepreUnroll];
#pragma unroll
            for (int u = 0; u < kRepreUnroll; ++u) { v[u] = ucm::gload16_nt(src + static_cast<size_t>(t + u) * row); }
#pragma unroll
            for (int u = 0; u < kRepreUnroll; ++u) { add_bf16x8(acc, v[u]); }
        }
        for (; t < merge; ++t) { add_bf16x8(acc, ucm::gload16_nt(src + static_cast<size_t>(t) * row)); }
        u32x4 o;
        o.x = mean_to_f16x2(acc[0], acc[1], inv);
        o.y = mean_to_f16x2(acc[2], acc[3], inv);
        o.z = mean_to_f16x2(acc[4], acc[5], inv);
        o.w = mean_to_f16x2(acc[6], acc[7], inv);
        *reinterpret_cast<u32x4*>(&stage[m * row + cg * 8]) = o;
    }
    __syncthreads();
    const unsigned pieces = d_pad / 8;
    unsigned short* out = repre + static_cast<int64_t>(blockIdx.y) * layer_stride + static_cast<size_t>(slot) * M * d_pad;
    for (unsigned e = threadIdx.x; e < kv_heads * pieces * M; e += kThreads) {
        const unsigned h = e / (pieces * M), rem = e - h * (pieces * M);
        const unsigned piece = rem / M, m = rem - piece * M;
        const unsigned short* srow = stage + m * row + h * head_dim;
        unsigned short c[8];
#pragma unroll
        for (unsigned j = 0; j < 8; ++j) {
            const unsigned p = piece * 8 + j;
            unsigned short v = 0;
            if (p < d_pruned) {
                const unsigned d = pruned ? static_cast<unsigned>(pruned[h * d_pruned + p]) : p;
                if (d < head_dim) { v = srow[d]; }
            }
            c[j] = v;
        }
        u32x4 o;
        o.x = c[0] | (static_cast<unsigned>(c[1]) << 16);
        o.y = c[2] | (static_cast<unsigned>(c[3]) << 16);
        o.z = c[4] | (static_cast<unsigned>(c[5]) << 16);
        o.w = c[6] | (static_cast<unsigned>(c[7]) << 16);
        ucm::gstore16(out + static_cast<int64_t>(h) * head_stride + static_cast<size_t>(rem) * 8, o);
    }
}

// ---- scores -> per-tile row maxima and per-block partial sums ------------------------------------
struct Task {
    const unsigned short* q;     // [tokens][q_heads][d_orig] of this task
    const int32_t* pruned;       // [kv_heads][d_pruned] or null
    const unsigned short* table; // first representative of the task: [n_blocks][M][kv_heads][d_pad]
    unsigned n_blocks;
};

template <int kM>
__device__ __forceinline__ void block_sums(const float (&e)[16], int half, float* __restrict__ prow, unsigned row_pad,
                                           unsigned blk0, unsigned n_blocks)
{
    // prow points at this lane's row inside block 0 of the [block][row_pad] plane: the 32 rows of one
    // block are one 128-byte line, written by one store instruction
    // e[i] belongs to sub-block (i/4)*8 + half*4 + i%4 of the tile
    float p4[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) { p4[g] = (e[4 * g] + e[4 * g + 1]) + (e[4 * g + 2] + e[4 * g + 3]); }
    if constexpr (kM >= 8) {
        constexpr int kGroups = kM / 8;                  // 8-sub-block groups per block
        constexpr int kBlocks = 4 / kGroups;             // blocks per tile
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
            float s = 0.0f;
#pragma unroll
            for (int g = 0; g < kGroups; ++g) { s += p4[b * kGroups + g]; }
            s += __shfl_xor(s, 32, 64);
            if (half == 0 && blk0 + b < n_blocks) { prow[static_cast<size_t>(blk0 + b) * row_pad] = s; }
        }
    } else if constexpr (kM == 4) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const unsigned b = blk0 + 2 * g + half;
            if (b < n_blocks) { prow[static_cast<size_t>(b) * row_pad] = p4[g]; }
        }
    } else if constexpr (kM == 2) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const unsigned b = blk0 + 4 * g + 2 * half;
            if (b < n_blocks) { prow[static_cast<size_t>(b) * row_pad] = e[4 * g] + e[4 * g + 1]; }
            if (b + 1 < n_blocks) { prow[static_cast<size_t>(b + 1) * row_pad] = e[4 * g + 2] + e[4 * g + 3]; }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const unsigned b = blk0 + (i >> 2) * 8 + half * 4 + (i & 3);
            if (b < n_blocks) { prow[static_cast<size_t>(b) * row_pad] = e[i]; }
        }
    }
}

// grid: x = chunk of sub-blocks, y = group of kv heads, z = task.  The table is head-major and
// piece-interleaved inside a block (see above), so what one workgroup streams for a head is one
// contiguous run read in whole lines (in the reference's [row][sub-block][kv head][d] order each
// vector of a head sits kv_heads*d*2 bytes from the next).  The queries of the group's heads are
// staged in LDS once per workgroup.
template <int kM, bool kTwoRowTiles>
__global__ __launch_bounds__(kThreads, kTwoRowTiles ? 2 : 3) void kvstar_score_kernel(
    const unsigned short* __restrict__ q, const int64_t* __restrict__ q_off, unsigned n_tokens, unsigned q_heads,
    unsigned d_orig, const int32_t* __restrict__ pruned, const int32_t* __restrict__ pruned_sel,
    const unsigned short* __restrict__ table, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, unsigned kv_heads, unsigned d_pruned, unsigned d_pad, int64_t head_stride,
    float* __restrict__ ws_max, float* __restrict__ ws_part, unsigned max_blocks, unsigned max_tiles,
    unsigned tiles_per_wave, unsigned row_pad, unsigned heads_per_group)
{
    extern __shared__ __attribute__((aligned(16))) unsigned short q_s[];   // [heads_per_group][row_pad][kQStride]

    const unsigned task = blockIdx.z;
    const unsigned h_first = blockIdx.y * heads_per_group;
    const unsigned nh = min(heads_per_group, kv_heads - h_first);
    const unsigned n_blocks = static_cast<unsigned>(max(seg_len[task], 0));
    const unsigned S = n_blocks * kM;
    const unsigned chunk = kWaves * tiles_per_wave * kTileSub;
    const unsigned s_chunk = blockIdx.x * chunk;
    if (s_chunk >= S) { return; }
    const unsigned g = q_heads / kv_heads, R = n_tokens * g;
    const int32_t psel = pruned_sel ? pruned_sel[task] : -1;
    const int32_t* pr0 = (pruned && psel >= 0) ? pruned + static_cast<size_t>(psel) * kv_heads * d_pruned : nullptr;

    // ---- the group's query rows, gathered by the kept channels, zero padded (rows up to row_pad, columns up to d_pad)
    const unsigned short* qt = q + q_off[task];
    if (!pr0 && d_pruned == d_pad && (d_orig % 8) == 0 && (reinterpret_cast<uintptr_t>(qt) & 15u) == 0) {
        const unsigned cpr = d_pad / 8;                  // 16-byte pieces per row
        for (unsigned e = threadIdx.x; e < nh * row_pad * cpr; e += kThreads) {
            const unsigned hr = e / cpr, c = e - hr * cpr;
            const unsigned hh = hr / row_pad, rho = hr - hh * row_pad;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (rho < R) {
                const unsigned xt = rho / g, gg = rho - xt * g;
                v = ucm::gload16(qt + (static_cast<size_t>(xt) * q_heads + (h_first + hh) * g + gg) * d_orig + c * 8);
            }
            *reinterpret_cast<u32x4*>(&q_s[hr * kQStride + c * 8]) = v;
        }
    } else {
        for (unsigned e = threadIdx.x; e < nh * row_pad * d_pad; e += kThreads) {
            const unsigned hr = e / d_pad, p = e - hr * d_pad;
            const unsigned hh = hr / row_pad, rho = hr - hh * row_pad;
            unsigned short v = 0;
            if (rho < R && p < d_pruned) {
                const unsigned xt = rho / g, gg = rho - xt * g;
                const unsigned d = pr0 ? static_cast<unsigned>(pr0[(h_first + hh) * d_pruned + p]) : p;
                if (d < d_orig) { v = qt[(static_cast<size_t>(xt) * q_heads + (h_first + hh) * g + gg) * d_orig + d]; }
            }
            q_s[hr * kQStride + p] = v;
        }
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = lane >> 5, lr = lane & 31;
    const unsigned ksteps = d_pad / 16;                  // MFMA steps; lane half `half`, step ks takes piece 2*ks + half
    const unsigned hoff = half * 8;
    constexpr bool two_row_tiles = kTwoRowTiles;   // 33..64 query rows per kv head
    // head-major table: head h's vectors of all sub-blocks are contiguous, d_pad elements each
    const unsigned short* tbase = table + static_cast<int64_t>(h_first) * head_stride +
                                  static_cast<size_t>(seg_off[task]) * kM * d_pad + half * (8 * kM);

    // A (tile, head) step's keys: eight 16-byte loads per lane, piece 2*ks + half of its sub-block; the
    // lanes of one instruction cover M*16 contiguous bytes per block and lane half.  Everything is
    // unconditional - MFMA steps past d_pad reload piece 0 and are multiplied with a zero query fragment,
    // lanes and tiles past the end reload the last vector and are masked - so that the loads of the NEXT
    // step can be issued before this step's arithmetic without a branch around them.
    auto load_keys = [&](u32x4 (&kf)[kMaxDim / 16], unsigned s0, unsigned hh) {
        const unsigned s_mine = min(s0 + lr, S - 1);
        const unsigned short* krow = tbase + static_cast<int64_t>(hh) * head_stride +
                                     static_cast<size_t>(s_mine / kM) * (kM * d_pad) + (s_mine % kM) * 8;
#pragma unroll
        for (unsigned ks = 0; ks < kMaxDim / 16; ++ks) { kf[ks] = ucm::gload16(krow + (ks < ksteps ? ks : 0u) * (16 * kM)); }
    };
    u32x4 kf[kMaxDim / 16], kn[kMaxDim / 16];
    const unsigned t_end = kWaves * tiles_per_wave;
    unsigned rot = (wave * 3u + blockIdx.x + task) % nh;
    load_keys(kf, s_chunk + wave * kTileSub, rot);
    for (unsigned t = wave; t < t_end; t += kWaves, rot = (rot + 1) % nh) {
        const unsigned s0 = s_chunk + t * kTileSub;
        if (s0 >= S) { break; }
        const unsigned tile = s0 / kTileSub;
        for (unsigned hi = 0; hi < nh; ++hi) {
            // heads are visited in an order rotated per wave and tile, so that the waves of a workgroup
            // are not all inside the same head's plane at once
            const unsigned hh = (hi + rot) % nh;
            {   // one load site (selects, no branch): the next head of this tile, or the first head of the wave's next tile
                const bool last = hi + 1 == nh;
                load_keys(kn, last ? s0 + kWaves * kTileSub : s0, (last ? rot + 1 : hi + 1 + rot) % nh);
            }
            const unsigned short* qh = q_s + static_cast<size_t>(hh) * row_pad * kQStride;
            const u32x4 zero = {0u, 0u, 0u, 0u};
            f32x16 acc0, acc1;
#pragma unroll
            for (int i = 0; i < 16; ++i) { acc0[i] = 0.0f; acc1[i] = 0.0f; }
#pragma unroll
            for (unsigned ks = 0; ks < kMaxDim / 16; ++ks) {
                const unsigned col = hoff + (ks < ksteps ? ks : 0u) * 16;
                const u32x4 braw = *reinterpret_cast<const u32x4*>(&qh[lr * kQStride + col]);
                const f16x8 b0 = __builtin_bit_cast(f16x8, ks < ksteps ? braw : zero);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kf[ks]), b0, acc0, 0, 0, 0);
            }
            if (two_row_tiles) {
#pragma unroll
                for (unsigned ks = 0; ks < kMaxDim / 16; ++ks) {
                    const unsigned col = hoff + (ks < ksteps ? ks : 0u) * 16;
                    const u32x4 braw = *reinterpret_cast<const u32x4*>(&qh[(32 + lr) * kQStride + col]);
                    const f16x8 b1 = __builtin_bit_cast(f16x8, ks < ksteps ? braw : zero);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kf[ks]), b1, acc1, 0, 0, 0);
                }
            }
            float* wmax = ws_max + (static_cast<size_t>(task) * kv_heads + h_first + hh) * row_pad * max_tiles;
            float* wpart = ws_part + (static_cast<size_t>(task) * kv_heads + h_first + hh) * row_pad * max_blocks;
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (rt == 1 && !two_row_tiles) { break; }
                const unsigned rho = rt * 32 + lr;
                float sc[16];
                float mx = -INFINITY;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const unsigned s = s0 + (i >> 2) * 8 + half * 4 + (i & 3);
                    const float v = rt == 0 ? acc0[i] : acc1[i];
                    sc[i] = s < S ? v : -INFINITY;
                    mx = fmaxf(mx, sc[i]);
                }
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));  // the tile has at least one live sub-block, so mx is finite
                float e[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) { e[i] = __expf(sc[i] - mx); }
                // rows past R hold zero queries: they are computed like the rest and never read
                if (half == 0) { wmax[static_cast<size_t>(tile) * row_pad + rho] = mx; }
                block_sums<kM>(e, half, wpart + rho, row_pad, s0 / kM, n_blocks);
            }
#pragma unroll
            for (unsigned ks = 0; ks < kMaxDim / 16; ++ks) { kf[ks] = kn[ks]; }
        }
    }
}

// ---- votes: rescale to the row maximum, normalise, add the rows ---------------------------------------
// The workspace planes of a (task, kv head) are [tile][row_pad] (tile maxima) and [block][row_pad]
// (partial sums): the rows of one tile or block are adjacent, so the score kernel's stores and the
// loads below move whole 128-byte lines.
//
// Phase 1, grid: x = kv head, y = task; thread = (group of tiles/blocks, row).  The row's global maximum
// and softmax denominator are reduced over its tiles, and each tile maximum in the workspace is
// replaced by the factor exp(tile max - row max) / denominator its partial sums have to be multiplied
// with.  Rows past tokens*group hold zero queries and are carried along.
__global__ __launch_bounds__(kThreads) void kvstar_rowscale_kernel(
    float* __restrict__ ws_max, const float* __restrict__ ws_part, const int32_t* __restrict__ seg_len,
    unsigned kv_heads, unsigned M, unsigned max_blocks, unsigned max_tiles, unsigned row_pad)
{
    __shared__ float red[kThreads];
    const unsigned task = blockIdx.y, h = blockIdx.x;
    const unsigned n_blocks = static_cast<unsigned>(max(seg_len[task], 0));
    if (n_blocks == 0) { return; }
    const unsigned n_tiles = (n_blocks * M + kTileSub - 1) / kTileSub;
    const unsigned rho = threadIdx.x % row_pad, grp = threadIdx.x / row_pad, ngrp = kThreads / row_pad;
    float* tm = ws_max + (static_cast<size_t>(task) * kv_heads + h) * row_pad * max_tiles + rho;
    const float* pp = ws_part + (static_cast<size_t>(task) * kv_heads + h) * row_pad * max_blocks + rho;
    float mx = -INFINITY;
    for (unsigned t = grp; t < n_tiles; t += ngrp) { mx = fmaxf(mx, tm[static_cast<size_t>(t) * row_pad]); }
    red[threadIdx.x] = mx;
    __syncthreads();
    mx = red[rho];
    for (unsigned g = 1; g < ngrp; ++g) { mx = fmaxf(mx, red[g * row_pad + rho]); }
    __syncthreads();
    float den = 0.0f;
    for (unsigned b = grp; b < n_blocks; b += ngrp) {
        den += pp[static_cast<size_t>(b) * row_pad] * __expf(tm[static_cast<size_t>((b * M) / kTileSub) * row_pad] - mx);
    }
    red[threadIdx.x] = den;
    __syncthreads();   // also: every read of the tile maxima above precedes the writes below
    den = red[rho];
    for (unsigned g = 1; g < ngrp; ++g) { den += red[g * row_pad + rho]; }
    const float inv = den > 1e-9f ? 1.0f / den : 1.0f;   // the reference skips the division then
    for (unsigned t = grp; t < n_tiles; t += ngrp) {
        tm[static_cast<size_t>(t) * row_pad] = __expf(tm[static_cast<size_t>(t) * row_pad] - mx) * inv;
    }
}

// Phase 2, grid: x = 8 blocks of the task, y = task; 32 lanes per block: votes[b] = sum over kv heads and
// rows of partial * factor.
__global__ __launch_bounds__(kThreads) void kvstar_vote_kernel(
    const float* __restrict__ ws_max, const float* __restrict__ ws_part, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, unsigned R, unsigned kv_heads, unsigned M, unsigned max_blocks,
    unsigned max_tiles, unsigned row_pad, float* __restrict__ votes)
{
    const unsigned task = blockIdx.y;
    const unsigned n_blocks = static_cast<unsigned>(max(seg_len[task], 0));
    if (blockIdx.x * 8 >= n_blocks) { return; }
    const unsigned b = blockIdx.x * 8 + (threadIdx.x >> 5), l32 = threadIdx.x & 31;
    const bool live = b < n_blocks;
    const unsigned tile = (b * M) / kTileSub;
    float v = 0.0f;
    if (live) {
        for (unsigned h = 0; h < kv_heads; ++h) {
            const float* wpart = ws_part + ((static_cast<size_t>(task) * kv_heads + h) * max_blocks + b) * row_pad;
            const float* wfac = ws_max + ((static_cast<size_t>(task) * kv_heads + h) * max_tiles + tile) * row_pad;
            for (unsigned rho = l32; rho < R; rho += 32) { v += wpart[rho] * wfac[rho]; }
        }
    }
#pragma unroll
    for (int d = 16; d >= 1; d >>= 1) { v += __shfl_xor(v, d, 64); }
    if (live && l32 == 0) { votes[seg_off[task] + b] = v; }
}

unsigned g_heads_per_group = 1;

}  // namespace

// Tuning knob for benchmarks: kv heads one workgroup of the KVStar score kernel walks (default 1).
extern "C" int ucm_set_kvstar_heads_per_group(int heads)
{
    UCM_REQUIRE(heads >= 1 && heads <= 8, "ucm_set_kvstar_heads_per_group: %d", heads);
    g_heads_per_group = static_cast<unsigned>(heads);
    return UCM_OK;
}

extern "C" int ucm_kvstar_block_repre(const void* const* k_layers, int n_layers, int num_blocks,
                                      const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                      int kv_heads, int head_dim, int merge, const int32_t* pruned, int d_pruned,
                                      int d_pad, void* repre_f16, int repre_rows, int64_t repre_layer_stride,
                                      int64_t repre_head_stride, ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0, "ucm_kvstar_block_repre: n=%d", n);
    if (n == 0) { return UCM_OK; }
    UCM_REQUIRE(k_layers && block_ids && slots && repre_f16, "ucm_kvstar_block_repre: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers <= 65535 && num_blocks > 0 && repre_rows > 0 && block_size > 0 && kv_heads > 0 &&
                    head_dim > 0, "ucm_kvstar_block_repre: non-positive shape");
    UCM_REQUIRE(merge > 0 && block_size % merge == 0, "ucm_kvstar_block_repre: merge=%d does not divide block_size=%d",
                merge, block_size);
    UCM_REQUIRE(d_pruned > 0 && d_pruned <= head_dim && d_pad >= d_pruned, "ucm_kvstar_block_repre: d_pruned=%d d_pad=%d",
                d_pruned, d_pad);
    UCM_REQUIRE(pruned || d_pruned == head_dim, "ucm_kvstar_block_repre: d_pruned < head_dim needs the channel list");
    const int M = block_size / merge;
    UCM_REQUIRE(repre_head_stride >= static_cast<int64_t>(repre_rows) * M * d_pad,
                "ucm_kvstar_block_repre: repre_head_stride=%lld smaller than one head's plane",
                static_cast<long long>(repre_head_stride));
    const unsigned row = static_cast<unsigned>(kv_heads) * static_cast<unsigned>(head_dim);
    UCM_SUPPORTED(row % 8 == 0 && d_pad % 8 == 0, "ucm_kvstar_block_repre: kv_heads*head_dim=%u and d_pad=%d must be multiples of 8",
                  row, d_pad);
    const size_t lds_bytes = static_cast<size_t>(M) * row * 2;
    UCM_SUPPORTED(lds_bytes <= 64u * 1024u, "ucm_kvstar_block_repre: %d sub-blocks of %u channels exceed 64 KiB of LDS", M, row);
    UCM_REQUIRE(ucm::aligned16(repre_f16) && repre_layer_stride % 8 == 0 && repre_head_stride % 8 == 0,
                "ucm_kvstar_block_repre: table not 16-byte aligned");
    if (lds_bytes > 48u * 1024u) {
        const hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(kvstar_repre_kernel),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
        if (ea != hipSuccess) { return ucm::check_hip(ea, "ucm_kvstar_block_repre (LDS size)"); }
    }
    hipLaunchKernelGGL(kvstar_repre_kernel, dim3(static_cast<unsigned>(n), n_layers), dim3(kThreads), lds_bytes,
                       ucm::as_stream(stream), k_layers, block_ids, slots, static_cast<unsigned>(num_blocks),
                       static_cast<unsigned>(repre_rows), static_cast<unsigned>(block_size),
                       static_cast<unsigned>(kv_heads), static_cast<unsigned>(head_dim), static_cast<unsigned>(merge),
                       pruned, static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad),
                       static_cast<unsigned short*>(repre_f16), repre_layer_stride, repre_head_stride);
    UCM_LAUNCH_CHECK("ucm_kvstar_block_repre");
}

extern "C" int ucm_kvstar_workspace_floats(int n_tasks, int kv_heads, int rows_per_head, int max_blocks, int sub_blocks,
                                           int64_t* max_floats, int64_t* part_floats)
{
    UCM_REQUIRE(n_tasks >= 0 && kv_heads > 0 && rows_per_head > 0 && rows_per_head <= kMaxRows && max_blocks >= 0 &&
                    sub_blocks > 0 && max_floats && part_floats, "ucm_kvstar_workspace_floats: bad argument");
    const int64_t tiles = (static_cast<int64_t>(max_blocks) * sub_blocks + kTileSub - 1) / kTileSub;
    const int64_t row_pad = rows_per_head > 32 ? 64 : 32;
    *max_floats = static_cast<int64_t>(n_tasks) * kv_heads * row_pad * std::max<int64_t>(tiles, 1);
    *part_floats = static_cast<int64_t>(n_tasks) * kv_heads * row_pad * std::max(max_blocks, 1);
    return UCM_OK;
}

extern "C" int ucm_kvstar_votes(const void* q_f16, const int64_t* q_off, int n_tokens, int q_heads, int d_orig,
                                const int32_t* pruned, const int32_t* pruned_sel, const void* repre_f16,
                                int64_t repre_head_stride, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                                int max_blocks,
                                int sub_blocks, int kv_heads, int d_pruned, int d_pad, float* ws_max, float* ws_part,
                                float* votes, ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks >= 0 && max_blocks >= 0, "ucm_kvstar_votes: n_tasks=%d max_blocks=%d", n_tasks, max_blocks);
    if (n_tasks == 0 || max_blocks == 0) { return UCM_OK; }
    UCM_REQUIRE(q_f16 && q_off && repre_f16 && seg_off && seg_len && ws_max && ws_part && votes, "ucm_kvstar_votes: null pointer");
    UCM_REQUIRE(n_tasks <= 65535, "ucm_kvstar_votes: n_tasks=%d", n_tasks);
    UCM_REQUIRE(kv_heads > 0 && q_heads >= kv_heads && q_heads % kv_heads == 0, "ucm_kvstar_votes: q_heads=%d kv_heads=%d",
                q_heads, kv_heads);
    UCM_SUPPORTED(kv_heads <= 8, "ucm_kvstar_votes: kv_heads=%d (at most 8)", kv_heads);
    UCM_REQUIRE(n_tokens > 0, "ucm_kvstar_votes: n_tokens=%d", n_tokens);
    UCM_SUPPORTED(n_tokens * (q_heads / kv_heads) <= kMaxRows, "ucm_kvstar_votes: tokens*group=%d (at most %d)",
                  n_tokens * (q_heads / kv_heads), kMaxRows);
    UCM_SUPPORTED(d_pad % 16 == 0 && d_pad > 0 && d_pad <= kMaxDim, "ucm_kvstar_votes: d_pad=%d (multiple of 16, at most %d)",
                  d_pad, kMaxDim);
    UCM_REQUIRE(d_pruned > 0 && d_pruned <= d_pad && d_pruned <= d_orig, "ucm_kvstar_votes: d_pruned=%d", d_pruned);
    UCM_REQUIRE(pruned_sel == nullptr || pruned != nullptr, "ucm_kvstar_votes: pruned_sel without pruned");
    UCM_REQUIRE(pruned_sel != nullptr || d_pruned == d_orig, "ucm_kvstar_votes: d_pruned < d_orig needs the channel lists");
    UCM_SUPPORTED(sub_blocks == 1 || sub_blocks == 2 || sub_blocks == 4 || sub_blocks == 8 || sub_blocks == 16 ||
                      sub_blocks == 32, "ucm_kvstar_votes: sub_blocks=%d (1, 2, 4, 8, 16 or 32)", sub_blocks);
    UCM_REQUIRE(ucm::aligned16(repre_f16) && repre_head_stride % 8 == 0 && repre_head_stride > 0,
                "ucm_kvstar_votes: representatives not 16-byte aligned");
    const int64_t S = static_cast<int64_t>(max_blocks) * sub_blocks;
    const unsigned max_tiles = static_cast<unsigned>((S + kTileSub - 1) / kTileSub);
    const unsigned R = static_cast<unsigned>(n_tokens * (q_heads / kv_heads));
    const unsigned row_pad = R > 32 ? 64 : 32;
    // heads per workgroup (at most what fits 72 KiB of LDS: 8 at 32 rows per head, 4 at 64); one by default,
    // ucm_set_kvstar_heads_per_group changes it
    const unsigned per_head_lds = row_pad * kQStride * 2;
    const unsigned heads_per_group = std::max(1u, std::min<unsigned>(std::min<unsigned>(kv_heads, g_heads_per_group),
                                                                     (72u * 1024u) / per_head_lds));
    const unsigned head_groups = (kv_heads + heads_per_group - 1) / heads_per_group;
    const unsigned lds_bytes = heads_per_group * per_head_lds;
    // a workgroup stages its queries once, so it should walk many tiles; the longest task is still cut into
    // enough chunks that about 2048 workgroups exist
    const unsigned tiles_per_wg_all = (max_tiles + kWaves - 1) / kWaves;
    const unsigned want_chunks = std::max(1u, 2048u / static_cast<unsigned>(n_tasks * head_groups));
    const unsigned tiles_per_wave = std::max(1u, (tiles_per_wg_all + want_chunks - 1) / want_chunks);
    const unsigned chunks = (max_tiles + kWaves * tiles_per_wave - 1) / (kWaves * tiles_per_wave);
    hipStream_t s = ucm::as_stream(stream);
#define UCM_KVSTAR_ARGS dim3(chunks, head_groups, n_tasks), dim3(kThreads), lds_bytes, s, static_cast<const unsigned short*>(q_f16), q_off, \
        static_cast<unsigned>(n_tokens), static_cast<unsigned>(q_heads), static_cast<unsigned>(d_orig), pruned, pruned_sel,   \
        static_cast<const unsigned short*>(repre_f16), seg_off, seg_len, static_cast<unsigned>(kv_heads),                     \
        static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad), repre_head_stride, ws_max, ws_part,                   \
        static_cast<unsigned>(max_blocks),                                                                                   \
        max_tiles, tiles_per_wave, row_pad, heads_per_group
#define UCM_KVSTAR_LAUNCH2(M, TWO)                                                                                    \
    do {                                                                                                             \
        if (lds_bytes > 48u * 1024u) {                                                                               \
            const hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(kvstar_score_kernel<M, TWO>),   \
                                                      hipFuncAttributeMaxDynamicSharedMemorySize,                   \
                                                      static_cast<int>(lds_bytes));                                \
            if (ea != hipSuccess) { return ucm::check_hip(ea, "ucm_kvstar_votes (LDS size)"); }                      \
        }                                                                                                            \
        hipLaunchKernelGGL((kvstar_score_kernel<M, TWO>), UCM_KVSTAR_ARGS);                                          \
    } while (0)
#define UCM_KVSTAR_LAUNCH(M)                                                                                          \
    do {                                                                                                             \
        if (R > 32) { UCM_KVSTAR_LAUNCH2(M, true); } else { UCM_KVSTAR_LAUNCH2(M, false); }                          \
    } while (0)
    switch (sub_blocks) {
    case 1: UCM_KVSTAR_LAUNCH(1); break;
    case 2: UCM_KVSTAR_LAUNCH(2); break;
    case 4: UCM_KVSTAR_LAUNCH(4); break;
    case 8: UCM_KVSTAR_LAUNCH(8); break;
    case 16: UCM_KVSTAR_LAUNCH(16); break;
    default: UCM_KVSTAR_LAUNCH(32); break;
    }
#undef UCM_KVSTAR_LAUNCH
#undef UCM_KVSTAR_LAUNCH2
#undef UCM_KVSTAR_ARGS
    if (hipError_t e = hipGetLastError(); e != hipSuccess) { return ucm::check_hip(e, "ucm_kvstar_votes (scores)"); }
    hipLaunchKernelGGL(kvstar_rowscale_kernel, dim3(static_cast<unsigned>(kv_heads), n_tasks), dim3(kThreads), 0, s, ws_max,
                       ws_part, seg_len, static_cast<unsigned>(kv_heads), static_cast<unsigned>(sub_blocks),
                       static_cast<unsigned>(max_blocks), max_tiles, row_pad);
    hipLaunchKernelGGL(kvstar_vote_kernel, dim3((max_blocks + 7) / 8, n_tasks), dim3(kThreads), 0, s, ws_max, ws_part, seg_off,
                       seg_len, R, static_cast<unsigned>(kv_heads), static_cast<unsigned>(sub_blocks),
                       static_cast<unsigned>(max_blocks), max_tiles, row_pad, votes);
    UCM_LAUNCH_CHECK("ucm_kvstar_votes");
}
