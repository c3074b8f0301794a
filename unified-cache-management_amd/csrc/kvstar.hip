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
constexpr int kTilesPerWave = 8;      // 32-sub-block tiles a wave walks per workgroup
constexpr int kChunk = kWaves * kTilesPerWave * 32;

__device__ __forceinline__ unsigned short f32_to_f16_bits(float f)
{
    const _Float16 h = static_cast<_Float16>(f);
    return __builtin_bit_cast(unsigned short, h);
}

// ---- sub-block representatives -------------------------------------------------------------
// grid: x = listed block * M + sub-block, y = layer; thread = (kv head, kept channel)
__global__ __launch_bounds__(kThreads) void kvstar_repre_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned rows, unsigned block_size, unsigned kv_heads,
    unsigned head_dim, unsigned merge, const int32_t* __restrict__ pruned, unsigned d_pruned, unsigned d_pad,
    unsigned short* __restrict__ repre, int64_t layer_stride)
{
    const unsigned M = block_size / merge;
    const unsigned item = blockIdx.x / M, m = blockIdx.x % M;
    const unsigned id = static_cast<unsigned>(block_ids[item]);
    const unsigned slot = static_cast<unsigned>(slots[item]);
    if (id >= num_blocks || slot >= rows) { return; }
    const unsigned row = kv_heads * head_dim;
    const unsigned short* blk = static_cast<const unsigned short*>(k_layers[blockIdx.y]) +
                                (static_cast<size_t>(id) * block_size + static_cast<size_t>(m) * merge) * row;
    unsigned short* out = repre + static_cast<int64_t>(blockIdx.y) * layer_stride +
                          (static_cast<size_t>(slot) * M + m) * kv_heads * d_pad;
    const float inv = 1.0f / static_cast<float>(merge);
    for (unsigned e = threadIdx.x; e < kv_heads * d_pad; e += kThreads) {
        const unsigned h = e / d_pad, p = e - h * d_pad;
        unsigned short v = 0;
        if (p < d_pruned) {
            const unsigned d = pruned ? static_cast<unsigned>(pruned[h * d_pruned + p]) : p;
            if (d < head_dim) {
                const UCM_GLOBAL unsigned short* src = (const UCM_GLOBAL unsigned short*)(blk + h * head_dim + d);
                float acc = __uint_as_float(static_cast<unsigned>(src[0]) << 16);
                for (unsigned t = 1; t < merge; ++t) {
                    acc = acc + __uint_as_float(static_cast<unsigned>(src[static_cast<size_t>(t) * row]) << 16);
                }
                acc = acc * inv;
                // to bf16 (round to nearest even), then to fp16: what mean() in the model dtype followed by .to(float16) gives
                unsigned u = __float_as_uint(acc);
                u += 0x7fffu + ((u >> 16) & 1u);
                v = f32_to_f16_bits(__uint_as_float(u & 0xffff0000u));
            }
        }
        out[e] = v;
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
__device__ __forceinline__ void block_sums(const float (&e)[16], int half, float* __restrict__ prow, unsigned blk0,
                                           unsigned n_blocks)
{
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
            if (half == 0 && blk0 + b < n_blocks) { prow[blk0 + b] = s; }
        }
    } else if constexpr (kM == 4) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const unsigned b = blk0 + 2 * g + half;
            if (b < n_blocks) { prow[b] = p4[g]; }
        }
    } else if constexpr (kM == 2) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const unsigned b = blk0 + 4 * g + 2 * half;
            if (b < n_blocks) { prow[b] = e[4 * g] + e[4 * g + 1]; }
            if (b + 1 < n_blocks) { prow[b + 1] = e[4 * g + 2] + e[4 * g + 3]; }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const unsigned b = blk0 + (i >> 2) * 8 + half * 4 + (i & 3);
            if (b < n_blocks) { prow[b] = e[i]; }
        }
    }
}

// grid: x = chunk of kChunk sub-blocks, y = kv head, z = task
template <int kM>
__global__ __launch_bounds__(kThreads) void kvstar_score_kernel(
    const unsigned short* __restrict__ q, const int64_t* __restrict__ q_off, unsigned n_tokens, unsigned q_heads,
    unsigned d_orig, const int32_t* __restrict__ pruned, const int32_t* __restrict__ pruned_sel,
    const unsigned short* __restrict__ table, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, unsigned kv_heads, unsigned d_pruned, unsigned d_pad,
    float* __restrict__ ws_max, float* __restrict__ ws_part, unsigned max_blocks, unsigned max_tiles)
{
    __shared__ __attribute__((aligned(16))) unsigned short q_s[kMaxRows * kQStride];

    const unsigned task = blockIdx.z, h = blockIdx.y;
    const unsigned n_blocks = static_cast<unsigned>(max(seg_len[task], 0));
    const unsigned S = n_blocks * kM;
    const unsigned s_chunk = blockIdx.x * kChunk;
    if (s_chunk >= S) { return; }
    const unsigned g = q_heads / kv_heads, R = n_tokens * g;
    const int32_t psel = pruned_sel ? pruned_sel[task] : -1;
    const int32_t* pr = (pruned && psel >= 0) ? pruned + (static_cast<size_t>(psel) * kv_heads + h) * d_pruned : nullptr;

    // ---- this head's query rows, gathered by the kept channels, zero padded
    const unsigned short* qt = q + q_off[task];
    for (unsigned e = threadIdx.x; e < kMaxRows * d_pad; e += kThreads) {
        const unsigned rho = e / d_pad, p = e - rho * d_pad;
        unsigned short v = 0;
        if (rho < R && p < d_pruned) {
            const unsigned xt = rho / g, gg = rho - xt * g;
            const unsigned d = pr ? static_cast<unsigned>(pr[p]) : p;
            if (d < d_orig) { v = qt[(static_cast<size_t>(xt) * q_heads + h * g + gg) * d_orig + d]; }
        }
        q_s[rho * kQStride + p] = v;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = lane >> 5, lr = lane & 31;
    const unsigned ksteps = d_pad / 16;                  // MFMA steps; lane half `half`, step ks takes dims half*(d_pad/2) + ks*8 .. +8
    const unsigned hoff = half * (d_pad / 2);
    const bool two_row_tiles = R > 32;
    const unsigned short* tbase = table + static_cast<size_t>(seg_off[task]) * kM * kv_heads * d_pad + static_cast<size_t>(h) * d_pad;
    const size_t vec_stride = static_cast<size_t>(kv_heads) * d_pad;

    float* wmax = ws_max + (static_cast<size_t>(task) * kv_heads + h) * kMaxRows * max_tiles;
    float* wpart = ws_part + (static_cast<size_t>(task) * kv_heads + h) * kMaxRows * max_blocks;

    for (unsigned t = wave; t < kWaves * kTilesPerWave; t += kWaves) {
        const unsigned s0 = s_chunk + t * 32;
        if (s0 >= S) { break; }
        const unsigned s_mine = min(s0 + lr, S - 1);     // clamp: lanes past the end read a valid vector and are masked below
        const unsigned short* krow = tbase + static_cast<size_t>(s_mine) * vec_stride + hoff;
        u32x4 kf[kMaxDim / 16];
#pragma unroll
        for (unsigned ks = 0; ks < kMaxDim / 16; ++ks) {
            if (ks < ksteps) { kf[ks] = ucm::gload16(krow + ks * 8); }
        }
        f32x16 acc0, acc1;
#pragma unroll
        for (int i = 0; i < 16; ++i) { acc0[i] = 0.0f; acc1[i] = 0.0f; }
#pragma unroll
        for (unsigned ks = 0; ks < kMaxDim / 16; ++ks) {
            if (ks < ksteps) {
                const f16x8 a = __builtin_bit_cast(f16x8, kf[ks]);
                const f16x8 b0 = *reinterpret_cast<const f16x8*>(&q_s[lr * kQStride + hoff + ks * 8]);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, acc0, 0, 0, 0);
                if (two_row_tiles) {
                    const f16x8 b1 = *reinterpret_cast<const f16x8*>(&q_s[(32 + lr) * kQStride + hoff + ks * 8]);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, acc1, 0, 0, 0);
                }
            }
        }
        const unsigned tile = s0 / 32;
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
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));      // the tile has at least one live sub-block, so mx is finite
            float e[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) { e[i] = __expf(sc[i] - mx); }
            // rows past R hold zero queries: they are computed like the rest and never read
            if (half == 0) { wmax[static_cast<size_t>(rho) * max_tiles + tile] = mx; }
            block_sums<kM>(e, half, wpart + static_cast<size_t>(rho) * max_blocks, s0 / kM, n_blocks);
        }
    }
}

// ---- votes: rescale to the row maximum, normalise, add the rows ---------------------------------------
// grid: x = task; one workgroup
__global__ __launch_bounds__(kThreads) void kvstar_combine_kernel(
    const float* __restrict__ ws_max, const float* __restrict__ ws_part, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, unsigned n_tokens, unsigned q_heads, unsigned kv_heads, unsigned M,
    unsigned max_blocks, unsigned max_tiles, float* __restrict__ votes)
{
    __shared__ float row_max[8 * kMaxRows];
    __shared__ float row_inv[8 * kMaxRows];
    const unsigned task = blockIdx.x;
    const unsigned n_blocks = static_cast<unsigned>(max(seg_len[task], 0));
    if (n_blocks == 0) { return; }
    const unsigned g = q_heads / kv_heads, R = n_tokens * g;
    const unsigned n_tiles = (n_blocks * M + 31) / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* wmax = ws_max + static_cast<size_t>(task) * kv_heads * kMaxRows * max_tiles;
    const float* wpart = ws_part + static_cast<size_t>(task) * kv_heads * kMaxRows * max_blocks;

    // one wave per (kv head, row): global maximum, then the softmax denominator
    for (unsigned row = wave; row < kv_heads * R; row += kWaves) {
        const unsigned h = row / R, rho = row - h * R;
        const float* tm = wmax + (static_cast<size_t>(h) * kMaxRows + rho) * max_tiles;
        const float* pp = wpart + (static_cast<size_t>(h) * kMaxRows + rho) * max_blocks;
        float mx = -INFINITY;
        for (unsigned t = lane; t < n_tiles; t += 64) { mx = fmaxf(mx, tm[t]); }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) { mx = fmaxf(mx, __shfl_xor(mx, d, 64)); }
        float den = 0.0f;
        for (unsigned b = lane; b < n_blocks; b += 64) { den += pp[b] * __expf(tm[(b * M) / 32] - mx); }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) { den += __shfl_xor(den, d, 64); }
        if (lane == 0) {
            row_max[h * kMaxRows + rho] = mx;
            row_inv[h * kMaxRows + rho] = den > 1e-9f ? 1.0f / den : 1.0f;   // the reference skips the division then
        }
    }
    __syncthreads();
    float* out = votes + seg_off[task];
    for (unsigned b = threadIdx.x; b < n_blocks; b += kThreads) {
        const unsigned tile = (b * M) / 32;
        float v = 0.0f;
        for (unsigned h = 0; h < kv_heads; ++h) {
            for (unsigned rho = 0; rho < R; ++rho) {
                const size_t r = static_cast<size_t>(h) * kMaxRows + rho;
                v += wpart[r * max_blocks + b] * __expf(wmax[r * max_tiles + tile] - row_max[h * kMaxRows + rho]) *
                     row_inv[h * kMaxRows + rho];
            }
        }
        out[b] = v;
    }
}

}  // namespace

extern "C" int ucm_kvstar_block_repre(const void* const* k_layers, int n_layers, int num_blocks,
                                      const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                      int kv_heads, int head_dim, int merge, const int32_t* pruned, int d_pruned,
                                      int d_pad, void* repre_f16, int repre_rows, int64_t repre_layer_stride,
                                      ucm_stream_t stream)
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
    UCM_REQUIRE(static_cast<int64_t>(n) * M <= 0x7fffffffll, "ucm_kvstar_block_repre: too many blocks for one launch");
    hipLaunchKernelGGL(kvstar_repre_kernel, dim3(static_cast<unsigned>(n) * M, n_layers), dim3(kThreads), 0,
                       ucm::as_stream(stream), k_layers, block_ids, slots, static_cast<unsigned>(num_blocks),
                       static_cast<unsigned>(repre_rows), static_cast<unsigned>(block_size),
                       static_cast<unsigned>(kv_heads), static_cast<unsigned>(head_dim), static_cast<unsigned>(merge),
                       pruned, static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad),
                       static_cast<unsigned short*>(repre_f16), repre_layer_stride);
    UCM_LAUNCH_CHECK("ucm_kvstar_block_repre");
}

extern "C" int ucm_kvstar_workspace_floats(int n_tasks, int kv_heads, int max_blocks, int sub_blocks, int64_t* max_floats,
                                           int64_t* part_floats)
{
    UCM_REQUIRE(n_tasks >= 0 && kv_heads > 0 && max_blocks >= 0 && sub_blocks > 0 && max_floats && part_floats,
                "ucm_kvstar_workspace_floats: bad argument");
    const int64_t tiles = (static_cast<int64_t>(max_blocks) * sub_blocks + 31) / 32;
    *max_floats = static_cast<int64_t>(n_tasks) * kv_heads * kMaxRows * std::max<int64_t>(tiles, 1);
    *part_floats = static_cast<int64_t>(n_tasks) * kv_heads * kMaxRows * std::max(max_blocks, 1);
    return UCM_OK;
}

extern "C" int ucm_kvstar_votes(const void* q_f16, const int64_t* q_off, int n_tokens, int q_heads, int d_orig,
                                const int32_t* pruned, const int32_t* pruned_sel, const void* repre_f16,
                                const int32_t* seg_off, const int32_t* seg_len, int n_tasks, int max_blocks,
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
    UCM_REQUIRE(ucm::aligned16(repre_f16), "ucm_kvstar_votes: representatives not 16-byte aligned");
    const int64_t S = static_cast<int64_t>(max_blocks) * sub_blocks;
    const unsigned chunks = static_cast<unsigned>((S + kChunk - 1) / kChunk);
    const unsigned max_tiles = static_cast<unsigned>((S + 31) / 32);
    hipStream_t s = ucm::as_stream(stream);
#define UCM_KVSTAR_ARGS dim3(chunks, kv_heads, n_tasks), dim3(kThreads), 0, s, static_cast<const unsigned short*>(q_f16), q_off, \
        static_cast<unsigned>(n_tokens), static_cast<unsigned>(q_heads), static_cast<unsigned>(d_orig), pruned, pruned_sel,   \
        static_cast<const unsigned short*>(repre_f16), seg_off, seg_len, static_cast<unsigned>(kv_heads),                     \
        static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad), ws_max, ws_part, static_cast<unsigned>(max_blocks),    \
        max_tiles
    switch (sub_blocks) {
    case 1: hipLaunchKernelGGL(kvstar_score_kernel<1>, UCM_KVSTAR_ARGS); break;
    case 2: hipLaunchKernelGGL(kvstar_score_kernel<2>, UCM_KVSTAR_ARGS); break;
    case 4: hipLaunchKernelGGL(kvstar_score_kernel<4>, UCM_KVSTAR_ARGS); break;
    case 8: hipLaunchKernelGGL(kvstar_score_kernel<8>, UCM_KVSTAR_ARGS); break;
    case 16: hipLaunchKernelGGL(kvstar_score_kernel<16>, UCM_KVSTAR_ARGS); break;
    default: hipLaunchKernelGGL(kvstar_score_kernel<32>, UCM_KVSTAR_ARGS); break;
    }
#undef UCM_KVSTAR_ARGS
    if (hipError_t e = hipGetLastError(); e != hipSuccess) { return ucm::check_hip(e, "ucm_kvstar_votes (scores)"); }
    hipLaunchKernelGGL(kvstar_combine_kernel, dim3(n_tasks), dim3(kThreads), 0, s, ws_max, ws_part, seg_off, seg_len,
                       static_cast<unsigned>(n_tokens), static_cast<unsigned>(q_heads), static_cast<unsigned>(kv_heads),
                       static_cast<unsigned>(sub_blocks), static_cast<unsigned>(max_blocks), max_tiles, votes);
    UCM_LAUNCH_CHECK("ucm_kvstar_votes");
}
