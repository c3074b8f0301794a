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
// halves.  What a tile leaves behind is 1/M of the score matrix, one number per
// (block, query row); it stays in LDS when a whole task fits there (the
// workgroup then finishes the votes of its kv head itself) and goes through a
// workspace in memory otherwise (two more kernels rescale to the global row
// maximum, normalise and add the rows up).  fp32 throughout; the summation
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
constexpr int64_t kLdsPathMinGroups = 128;            // (task, kv head) pairs from which the in-LDS path is taken
constexpr size_t kLdsPathMaxBytes = 159 * 1024;       // of the 160 KiB a compute unit has

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
// Phase 1: a thread owns 8 adjacent columns of a token row
// (one 16-byte load per token, `merge` tokens accumulated in token order in fp32), the means -
// rounded to bf16 and then fp16, what mean() in the model dtype followed by .to(float16) gives -
// are parked in LDS as [sub-block][kv_heads*head_dim] (as many sub-blocks at a time as fit 64 KiB).
// Phase 2 gathers the kept channels from LDS and writes the pieces, consecutive threads to consecutive
// 16 bytes.
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

// float16 keys: the mean is rounded once, to float16 - what mean() gives in a float16 model (the .to(float16) that
// follows changes nothing)
__device__ __forceinline__ unsigned mean_f16keys_to_f16x2(float lo, float hi, float inv)
{
    float a = lo * inv, b = hi * inv;
    asm volatile("" : "+v"(a), "+v"(b));     // the product is rounded to fp32 first, as torch's mean is, then converted
    return static_cast<unsigned>(f32_to_f16_bits(a)) | (static_cast<unsigned>(f32_to_f16_bits(b)) << 16);
}

__device__ __forceinline__ void add_f16x8(float (&acc)[8], const u32x4 v)
{
    const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        acc[2 * j] = acc[2 * j] + static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(w[j] & 0xffffu)));
        acc[2 * j + 1] = acc[2 * j + 1] + static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(w[j] >> 16)));
    }
}

template <bool kF16>
__device__ __forceinline__ void add_keys8(float (&acc)[8], const u32x4 v)
{
    if (kF16) { add_f16x8(acc, v); } else { add_bf16x8(acc, v); }
}

template <bool kF16>
__device__ __forceinline__ unsigned mean_pair(float lo, float hi, float inv)
{
    return kF16 ? mean_f16keys_to_f16x2(lo, hi, inv) : mean_to_f16x2(lo, hi, inv);
}


// With channel lists, which (kv head, 16-byte piece) pairs a thread writes is decided once per kernel when the
// pairs divide the workgroup: kThreads / pairs threads share a pair and split its sub-blocks, and the pair's eight
// kept channels stay in registers (-1: a padding column).  Reading the lists again for every piece and turning
// a flat index into (head, piece, sub-block) by division cost more instructions than the key loads themselves.
struct PieceMap {
    bool fixed;
    unsigned h, piece, sub, tpp;
    int d[8];
};

__device__ __forceinline__ PieceMap make_piece_map(const int32_t* __restrict__ lists, unsigned kv_heads, unsigned head_dim,
                                                   unsigned d_pruned, unsigned pieces)
{
    PieceMap m;
    const unsigned pairs = kv_heads * pieces;
    m.fixed = lists != nullptr && pairs <= static_cast<unsigned>(kThreads) && (kThreads % pairs) == 0;
    m.tpp = m.fixed ? kThreads / pairs : 1u;
    const unsigned pair = threadIdx.x / m.tpp;
    m.sub = threadIdx.x - pair * m.tpp;
    m.h = m.fixed ? pair / pieces : 0u;
    m.piece = m.fixed ? pair - m.h * pieces : 0u;
#pragma unroll
    for (unsigned j = 0; j < 8; ++j) {
        const unsigned p = m.piece * 8 + j;
        int d = -1;
        if (m.fixed && p < d_pruned) {
            d = lists[m.h * d_pruned + p];
            if (d < 0 || static_cast<unsigned>(d) >= head_dim) { d = -1; }
        }
        m.d[j] = d;
    }
    return m;
}

// Phase 2 of the representative kernels: the kept channels of the staged means of sub-blocks m0 .. m0+mc-1,
// gathered from LDS and written as the table's 16-byte pieces, consecutive threads to consecutive 16 bytes.
// The stores are non-temporal: the table is not read again by this kernel, and one byte written per eight read
// costs less that way (a plain streaming kernel with the same mix of 32.4 GB read and 4 GB written measures
// 6.6 ms with non-temporal stores and 7.0 ms with plain ones; this kernel 7.2 against 7.4).
__device__ __forceinline__ void repre_write_pieces(const unsigned short* __restrict__ stage, const int32_t* __restrict__ kept,
                                                   bool pruned, unsigned kv_heads, unsigned head_dim, unsigned d_pruned,
                                                   unsigned pieces, unsigned srow_stride, unsigned M, unsigned m0, unsigned mc,
                                                   unsigned short* __restrict__ out, int64_t head_stride, const PieceMap& pm)
{
    if (pm.fixed) {
        unsigned short* dst = out + static_cast<int64_t>(pm.h) * head_stride + (static_cast<size_t>(pm.piece) * M + m0) * 8;
        const unsigned short* src = stage + pm.h * head_dim;
        for (unsigned ml = pm.sub; ml < mc; ml += pm.tpp) {
            const unsigned short* srow = src + ml * srow_stride;
            unsigned short c[8];
#pragma unroll
            for (unsigned j = 0; j < 8; ++j) { c[j] = pm.d[j] >= 0 ? srow[pm.d[j]] : static_cast<unsigned short>(0); }
            u32x4 o;
            o.x = c[0] | (static_cast<unsigned>(c[1]) << 16);
            o.y = c[2] | (static_cast<unsigned>(c[3]) << 16);
            o.z = c[4] | (static_cast<unsigned>(c[5]) << 16);
            o.w = c[6] | (static_cast<unsigned>(c[7]) << 16);
            ucm::gstore16_nt(dst + static_cast<size_t>(ml) * 8, o);
        }
        return;
    }
    for (unsigned e = threadIdx.x; e < kv_heads * pieces * mc; e += kThreads) {
        const unsigned h = e / (pieces * mc), rem = e - h * (pieces * mc);
        const unsigned piece = rem / mc, ml = rem - piece * mc;
        const unsigned short* srow = stage + ml * srow_stride + h * head_dim;
        u32x4 o;
        if (!pruned && piece * 8 + 8 <= d_pruned) {      // all channels kept: the piece is 16 contiguous bytes
            o = *reinterpret_cast<const u32x4*>(srow + piece * 8);
        } else {
            unsigned short c[8];
#pragma unroll
            for (unsigned j = 0; j < 8; ++j) {
                const unsigned p = piece * 8 + j;
                unsigned short v = 0;
                if (p < d_pruned) {
                    const unsigned d = pruned ? static_cast<unsigned>(kept[h * d_pruned + p]) : p;
                    if (d < head_dim) { v = srow[d]; }
                }
                c[j] = v;
            }
            o.x = c[0] | (static_cast<unsigned>(c[1]) << 16);
            o.y = c[2] | (static_cast<unsigned>(c[3]) << 16);
            o.z = c[4] | (static_cast<unsigned>(c[5]) << 16);
            o.w = c[6] | (static_cast<unsigned>(c[7]) << 16);
        }
        ucm::gstore16_nt(out + static_cast<int64_t>(h) * head_stride + (static_cast<size_t>(piece) * M + m0 + ml) * 8, o);
    }
}

// Sub-blocks of 1, 2, 4 or 8 tokens (kMerge).  Workgroups are persistent over the list of cache blocks
// (grid: x = workgroup, stepping by the grid; y = layer) and the work of one is a sequence of UNITS: a unit
// is 16 loads of 16 bytes per thread - 16/kMerge (sub-block, 8 columns) items - of one chunk of one cache
// block.  The loads of the next unit - of the same chunk, the next chunk or the next cache block - are
// issued before the current unit's means are formed, so key loads stay in flight through the phase that
// writes a chunk's pieces out and across cache blocks.
template <int kMerge, bool kF16>
__global__ __launch_bounds__(kThreads) void kvstar_repre_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned n_items, unsigned rows, unsigned block_size,
    unsigned kv_heads, unsigned head_dim, const int32_t* __restrict__ pruned, int64_t pruned_layer_stride,
    const int32_t* __restrict__ list_sel, unsigned n_lists,
    unsigned d_pruned, unsigned d_pad, unsigned short* __restrict__ repre, int64_t layer_stride, int64_t head_stride,
    int64_t row_stride, unsigned m_chunk)
{
    static_assert(kMerge == 1 || kMerge == 2 || kMerge == 4 || kMerge == 8, "tokens per sub-block");
    extern __shared__ __attribute__((aligned(16))) unsigned short stage[];   // [m_chunk][row + 8]: the 16 bytes of padding
    constexpr unsigned kBatch = kRepreUnroll / kMerge;                       // spread the sub-blocks' rows over the LDS banks
    const unsigned M = block_size / kMerge;
    const unsigned row = kv_heads * head_dim, ncg = row / 8, srow_stride = row + 8;
    const float inv = 1.0f / static_cast<float>(kMerge);
    const unsigned pieces = d_pad / 8;
    const unsigned short* layer = static_cast<const unsigned short*>(k_layers[blockIdx.y]);
    // the channel lists, read once: a load from memory per output piece would queue behind the key stream
    int32_t* kept = reinterpret_cast<int32_t*>(stage + static_cast<size_t>(m_chunk) * srow_stride);
    const int32_t* my_lists = pruned ? pruned + static_cast<int64_t>(blockIdx.y) * pruned_layer_stride : nullptr;
    if (pruned) {   // this layer's lists (a stride of 0: one set of lists for every layer)
        for (unsigned e = threadIdx.x; e < kv_heads * d_pruned; e += kThreads) { kept[e] = my_lists[e]; }
    }
    PieceMap pm = make_piece_map(my_lists, kv_heads, head_dim, d_pruned, pieces);
    // list_sel: every listed block names the list of the layer's n_lists it is pruned by (the blocks of several
    // requests in one launch, each request with channels of its own); the list in use is replaced when a block
    // names another one, which is once per request and workgroup
    unsigned cur_list = 0;

    struct Unit {
        unsigned item, m0, w_first;                      // cache block in the list, first sub-block of the chunk, first work item
        unsigned wq, wr;                                 // w_first = wq * ncg + wr
        const unsigned short* blk;
        bool valid;
    };
    // (sub-block, column group) of a work item is its number divided by ncg.  One division per thread here and
    // additions with a carry afterwards: a division per load cost as many instructions as the means themselves.
    const unsigned tq = threadIdx.x / ncg, tr = threadIdx.x - tq * ncg;                 // this thread's offset inside a unit
    const unsigned sq = kThreads / ncg, sr = kThreads - sq * ncg;                        // step between a thread's items
    const unsigned uq = (kThreads * kBatch) / ncg, ur = kThreads * kBatch - uq * ncg;   // step between units
    auto step = [&](unsigned& q, unsigned& r, unsigned dq, unsigned dr) {
        q += dq;
        r += dr;
        if (r >= ncg) { r -= ncg; ++q; }
    };
    // first usable cache block at or after `from` (a block id or slot out of range is skipped, never dereferenced)
    auto seek = [&](Unit& u, unsigned from) {
        for (unsigned i = from; i < n_items; i += gridDim.x) {
            const unsigned id = static_cast<unsigned>(block_ids[i]);
            if (id < num_blocks && static_cast<unsigned>(slots[i]) < rows &&
                (!list_sel || static_cast<unsigned>(list_sel[i]) < n_lists)) {
                u.item = i;
                u.m0 = 0;
                u.w_first = 0;
                u.wq = u.wr = 0;
                u.blk = layer + static_cast<size_t>(id) * block_size * row;
                return;
            }
        }
        u.valid = false;
    };
    auto next_of = [&](const Unit& u) -> Unit {
        Unit n = u;
        const unsigned mc = min(m_chunk, M - u.m0);
        n.w_first = u.w_first + kThreads * kBatch;
        step(n.wq, n.wr, uq, ur);
        if (n.w_first >= mc * ncg) {
            n.w_first = 0;
            n.wq = n.wr = 0;
            n.m0 = u.m0 + m_chunk;
            if (n.m0 >= M) { seek(n, u.item + gridDim.x); }
        }
        return n;
    };
    // unconditional: work items past the chunk's end reload its last one
    auto load_unit = [&](u32x4 (&v)[kRepreUnroll], const Unit& u) {
        const unsigned mc = min(m_chunk, M - u.m0), last = mc * ncg - 1;
        unsigned q = u.wq, r = u.wr;
        step(q, r, tq, tr);
#pragma unroll
        for (unsigned j = 0; j < kBatch; ++j) {
            const bool past = u.w_first + threadIdx.x + j * kThreads > last;
            const unsigned ml = past ? mc - 1 : q, cg = past ? ncg - 1 : r;
            step(q, r, sq, sr);
            const unsigned short* src = u.blk + static_cast<size_t>(u.m0 + ml) * kMerge * row + cg * 8;
#pragma unroll
            for (unsigned t = 0; t < kMerge; ++t) { v[j * kMerge + t] = ucm::gload16_nt(src + static_cast<size_t>(t) * row); }
        }
        asm volatile("" ::: "memory");                   // keeps the compiler from sinking the loads to their use
    };
    // `live` false: the unit does not exist (the sequence has ended); its registers are still read, nothing is written
    auto finish_unit = [&](const u32x4 (&v)[kRepreUnroll], const Unit& u, bool live) {
        const unsigned mc = min(m_chunk, M - u.m0), n_work = live ? mc * ncg : 0u;
        unsigned q = u.wq, r = u.wr;
        step(q, r, tq, tr);
#pragma unroll
        for (unsigned j = 0; j < kBatch; ++j) {
            const unsigned w = u.w_first + threadIdx.x + j * kThreads;
            const unsigned ml = q, cg = r;
            step(q, r, sq, sr);
            // the means are formed whether or not the item exists: were the loaded registers read only under a
            // branch, the compiler could not tell further down that their loads have returned, and would wait
            // there for every load in flight, the next unit's included
            float acc[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) { acc[c] = -0.0f; }   // -0 + x == x for every x, signed zeros included
#pragma unroll
            for (unsigned t = 0; t < kMerge; ++t) { add_keys8<kF16>(acc, v[j * kMerge + t]); }
            u32x4 o;
            o.x = mean_pair<kF16>(acc[0], acc[1], inv);
            o.y = mean_pair<kF16>(acc[2], acc[3], inv);
            o.z = mean_pair<kF16>(acc[4], acc[5], inv);
            o.w = mean_pair<kF16>(acc[6], acc[7], inv);
            if (w < n_work) { *reinterpret_cast<u32x4*>(&stage[ml * srow_stride + cg * 8]) = o; }
        }
        if (live && u.w_first + kThreads * kBatch >= mc * ncg) { // the chunk is staged: write its pieces
            if (list_sel && static_cast<unsigned>(list_sel[u.item]) != cur_list) {      // (the same for all threads)
                cur_list = static_cast<unsigned>(list_sel[u.item]);
                const int32_t* lists = my_lists + static_cast<size_t>(cur_list) * kv_heads * d_pruned;
                __syncthreads();                         // nobody reads the old list any more
                for (unsigned e = threadIdx.x; e < kv_heads * d_pruned; e += kThreads) { kept[e] = lists[e]; }
                pm = make_piece_map(lists, kv_heads, head_dim, d_pruned, pieces);
            }
            __syncthreads();
            unsigned short* out = repre + static_cast<int64_t>(blockIdx.y) * layer_stride +
                                  static_cast<int64_t>(static_cast<unsigned>(slots[u.item])) * row_stride;
            repre_write_pieces(stage, kept, pruned != nullptr, kv_heads, head_dim, d_pruned, pieces, srow_stride, M, u.m0, mc,
                               out, head_stride, pm);
            __syncthreads();                             // the next chunk overwrites the staged means
        }
    };

    // Two units per round, one in each register set, and ONE way out of the loop, at its end: with a second exit
    // between the halves the compiler joins both exits in one block that also leads back to the loop's head, and
    // then waits at the head for the loads it believes may have just been issued - all of them, every round.
    Unit a{0u, 0u, 0u, 0u, 0u, nullptr, true};
    seek(a, blockIdx.x);
    if (!a.valid) { return; }                            // the whole workgroup: the unit sequence is the same for all threads
    u32x4 va[kRepreUnroll], vb[kRepreUnroll];
    load_unit(va, a);
    for (;;) {
        const Unit b = next_of(a);                       // past the end: a reloads (16 loads per workgroup, once)
        load_unit(vb, b.valid ? b : a);
        finish_unit(va, a, true);
        const Unit c = b.valid ? next_of(b) : b;
        load_unit(va, c.valid ? c : a);
        finish_unit(vb, b.valid ? b : a, b.valid);
        if (!c.valid) { break; }
        a = c;
    }
}

// Any other number of tokens per sub-block: one workgroup per cache block, the tokens of a sub-block summed
// sixteen loads at a time.  grid: x = cache block of the list, y = layer.
template <bool kF16>
__global__ __launch_bounds__(kThreads) void kvstar_repre_any_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned rows, unsigned block_size, unsigned kv_heads,
    unsigned head_dim, unsigned merge, const int32_t* __restrict__ pruned, int64_t pruned_layer_stride,
    const int32_t* __restrict__ list_sel, unsigned n_lists, unsigned d_pruned, unsigned d_pad,
    unsigned short* __restrict__ repre, int64_t layer_stride, int64_t head_stride, int64_t row_stride, unsigned m_chunk)
{
    extern __shared__ __attribute__((aligned(16))) unsigned short stage[];   // [m_chunk][row + 8]
    const unsigned M = block_size / merge;
    const unsigned id = static_cast<unsigned>(block_ids[blockIdx.x]);
    const unsigned slot = static_cast<unsigned>(slots[blockIdx.x]);
    const unsigned sel = list_sel ? static_cast<unsigned>(list_sel[blockIdx.x]) : 0u;
    if (id >= num_blocks || slot >= rows || (list_sel && sel >= n_lists)) { return; }   // whole workgroup: never dereference a bad id
    const unsigned row = kv_heads * head_dim, ncg = row / 8, srow_stride = row + 8;
    const unsigned short* blk = static_cast<const unsigned short*>(k_layers[blockIdx.y]) +
                                static_cast<size_t>(id) * block_size * row;
    const float inv = 1.0f / static_cast<float>(merge);
    const unsigned pieces = d_pad / 8;
    unsigned short* out = repre + static_cast<int64_t>(blockIdx.y) * layer_stride + static_cast<int64_t>(slot) * row_stride;
    int32_t* kept = reinterpret_cast<int32_t*>(stage + static_cast<size_t>(m_chunk) * srow_stride);
    // this layer's lists (a stride of 0: one set of lists for every layer), and of them the one the block names
    const int32_t* my_lists = pruned ? pruned + static_cast<int64_t>(blockIdx.y) * pruned_layer_stride +
                                           static_cast<size_t>(sel) * kv_heads * d_pruned : nullptr;
    if (pruned) {
        for (unsigned e = threadIdx.x; e < kv_heads * d_pruned; e += kThreads) { kept[e] = my_lists[e]; }
    }
    const PieceMap pm = make_piece_map(my_lists, kv_heads, head_dim, d_pruned, pieces);
    for (unsigned m0 = 0; m0 < M; m0 += m_chunk) {       // m_chunk sub-blocks at a time: what fits LDS
        const unsigned mc = min(m_chunk, M - m0);
        for (unsigned w = threadIdx.x; w < mc * ncg; w += kThreads) {
            const unsigned ml = w / ncg, cg = w - ml * ncg;
            const unsigned short* src = blk + static_cast<size_t>(m0 + ml) * merge * row + cg * 8;
            float acc[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) { acc[c] = -0.0f; }   // -0 + x == x for every x, signed zeros included
            unsigned t = 0;
            for (; t + kRepreUnroll <= merge; t += kRepreUnroll) {
                u32x4 v[kRepreUnroll];
#pragma unroll
                for (int u = 0; u < kRepreUnroll; ++u) { v[u] = ucm::gload16_nt(src + static_cast<size_t>(t + u) * row); }
#pragma unroll
                for (int u = 0; u < kRepreUnroll; ++u) { add_keys8<kF16>(acc, v[u]); }
            }
            for (; t < merge; ++t) { add_keys8<kF16>(acc, ucm::gload16_nt(src + static_cast<size_t>(t) * row)); }
            u32x4 o;
            o.x = mean_pair<kF16>(acc[0], acc[1], inv);
            o.y = mean_pair<kF16>(acc[2], acc[3], inv);
            o.z = mean_pair<kF16>(acc[4], acc[5], inv);
            o.w = mean_pair<kF16>(acc[6], acc[7], inv);
            *reinterpret_cast<u32x4*>(&stage[ml * srow_stride + cg * 8]) = o;
        }
        __syncthreads();
        repre_write_pieces(stage, kept, pruned != nullptr, kv_heads, head_dim, d_pruned, pieces, srow_stride, M, m0, mc, out,
                           head_stride, pm);
        __syncthreads();                                 // the next chunk overwrites the staged means
    }
}

// The two halves of a wave hold the two halves of every query row's tile: one v_permlane32_swap hands each
// lane its own and its partner's value (lower half's first), without a trip through LDS.
__device__ __forceinline__ float halves_max(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// kM here: sub-blocks per part (a block, or a tile's share of a bigger block; at most 32).
// Hands the per-block sums of a tile's 32 exponentials for this lane's row to put(block within the tile,
// sum) and returns their total (both lane halves included).  put is called unconditionally by all 64 lanes:
// a store the compiler has to branch around would make it wait for ALL outstanding memory operations.
template <int kM, typename Put>
__device__ __forceinline__ float block_sums(const float (&e)[16], int half, Put put)
{
    // e[i] belongs to sub-block (i/4)*8 + half*4 + i%4 of the tile
    float p4[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) { p4[g] = (e[4 * g] + e[4 * g + 1]) + (e[4 * g + 2] + e[4 * g + 3]); }
    if constexpr (kM >= 8) {
        constexpr int kGroups = kM / 8;                  // 8-sub-block groups per block
        constexpr int kBlocks = 4 / kGroups;             // blocks per tile
        float sum[kBlocks];
        float total = 0.0f;
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
            float v = 0.0f;
#pragma unroll
            for (int g = 0; g < kGroups; ++g) { v += p4[b * kGroups + g]; }
            sum[b] = halves_sum(v);                      // both halves now hold the block's sum
            total += sum[b];
        }
        if constexpr (kBlocks == 1) {
            put(0u, sum[0]);                             // the two halves put the same value in the same place
        } else {
#pragma unroll
            for (int j = 0; j < kBlocks / 2; ++j) {      // lower half: block 2j, upper half: block 2j+1
                put(static_cast<unsigned>(2 * j + half), half ? sum[2 * j + 1] : sum[2 * j]);
            }
        }
        return total;
    } else {
        if constexpr (kM == 4) {
#pragma unroll
            for (int g = 0; g < 4; ++g) { put(static_cast<unsigned>(2 * g + half), p4[g]); }
        } else if constexpr (kM == 2) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                put(static_cast<unsigned>(4 * g + 2 * half), e[4 * g] + e[4 * g + 1]);
                put(static_cast<unsigned>(4 * g + 2 * half + 1), e[4 * g + 2] + e[4 * g + 3]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) { put(static_cast<unsigned>((i >> 2) * 8 + half * 4 + (i & 3)), e[i]); }
        }
        float total = (p4[0] + p4[1]) + (p4[2] + p4[3]);
        total = halves_sum(total);
        return total;
    }
}

constexpr float kLog2e = 1.4426950408889634f;

// What bounds the descriptors a task brings in device memory: its rows inside the table / the votes array, its
// query block inside the query buffer, its channel list inside the lists.  A task outside any of them counts
// zero blocks in every kernel of the call, so none of its descriptors is followed and its votes stay as they were.
struct TaskBounds {
    int64_t rows_bound;     // rows of the shared table (ucm_kvstar_votes) and entries of `votes`
    int64_t q_elems;        // fp16 elements the query buffer holds
    int64_t q_need;         // elements a task reads from q_off[task] on: n_tokens * q_heads * d_orig
    int n_lists;            // channel lists in `pruned`
};

__device__ __forceinline__ unsigned task_blocks(const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len,
                                                const int64_t* __restrict__ q_off, const int32_t* __restrict__ pruned_sel,
                                                unsigned task, unsigned max_blocks, const TaskBounds& tb)
{
    const int n = min(max(seg_len[task], 0), static_cast<int>(max_blocks));   // the planes are sized for max_blocks
    const int64_t so = seg_off[task], qo = q_off[task];
    const bool ok = so >= 0 && so + n <= tb.rows_bound && qo >= 0 && qo + tb.q_need <= tb.q_elems &&
                    (!pruned_sel || pruned_sel[task] < tb.n_lists);
    return ok ? static_cast<unsigned>(n) : 0u;
}

// grid: x = chunk of sub-blocks, y = kv head, z = task.  The table is head-major and piece-interleaved
// inside a block (see above), so what one workgroup streams is one contiguous run read in whole lines
// (in the reference's [row][sub-block][kv head][d] order each vector of a head sits kv_heads*d*2 bytes
// from the next).  The head's query rows are staged in LDS once per workgroup.
//
// kSteps = MFMA steps a vector takes (d_pad <= 16*kSteps; 2, 4 or 8).  A wave always moves eight
// 16-byte loads per lane at a time - a "span" of 8/kSteps tiles of 32 sub-blocks - so the bytes in
// flight do not shrink with the vectors.
//
// kLds == false (any task length; a task may be cut into chunks): per tile and query row the kernel
// leaves the reference the tile's exponentials are relative to and their sum ([tile][2][row_pad]) and the per-block sums
// ([part][row_pad]; a part is a block, or a tile's share of a block of more than 32 sub-blocks) in the
// workspace for the two kernels below.
//
// kLds == true (one workgroup walks the whole task and the task's plane fits LDS): the plane stays in
// LDS, as log2 of each entry's sum of exponentials (one number instead of a sum and the maximum it is
// relative to; an entry is a block, or a span's share of a block longer than a span), the workgroup
// itself reduces every row's maximum and denominator when it is through, and only this head's share of
// the votes ([task][kv head][max_blocks], in ws_part) goes to memory: 1/32 of the other path's stores,
// whose number per compute unit - not their bytes - is what that path pays for.
template <int kM, int kSteps, bool kTwoRowTiles, bool kLds>
__global__ __launch_bounds__(kThreads, 2) void kvstar_score_kernel(
    const unsigned short* __restrict__ q, const int64_t* __restrict__ q_off, unsigned n_tokens, unsigned q_heads,
    unsigned d_orig, const int32_t* __restrict__ pruned, const int32_t* __restrict__ pruned_sel,
    const unsigned short* __restrict__ table, const void* const* __restrict__ task_tables,
    const int64_t* __restrict__ task_head_strides, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, unsigned kv_heads, unsigned d_pruned, unsigned d_pad, int64_t head_stride,
    int64_t row_stride, float* __restrict__ ws_max, float* __restrict__ ws_part, unsigned max_blocks, unsigned max_tiles,
    unsigned spans_per_wave, unsigned row_pad, unsigned plane_offset, unsigned q_full_ok, const TaskBounds tb)
{
    static_assert(kM >= 1 && kM <= 128 && (kM & (kM - 1)) == 0, "sub-blocks per block");
    static_assert(kSteps == 2 || kSteps == 4 || kSteps == 8, "MFMA steps per vector");
    constexpr int kLoads = kMaxDim / 16;                 // 16-byte loads per lane and span
    constexpr int kSpanTiles = kLoads / kSteps;
    constexpr unsigned kSpan = kSpanTiles * kTileSub;    // sub-blocks per span
    constexpr int kRowTiles = kTwoRowTiles ? 2 : 1;      // 33..64 query rows per kv head take two
    constexpr unsigned kStride = kWaves * kSpan;         // from one span of a wave to its next
    constexpr int kTilePart = kM < kTileSub ? kM : kTileSub;          // sub-blocks of one block inside one tile
    constexpr unsigned kPartsPerTile = kTileSub / kTilePart;
    constexpr unsigned kEntrySub = kM < static_cast<int>(kSpan) ? kM : kSpan;   // kLds: sub-blocks per plane entry
    constexpr unsigned kEntryTiles = kEntrySub > kTileSub ? kEntrySub / kTileSub : 1;
    constexpr unsigned kEntriesPerBlock = kM / kEntrySub;

    extern __shared__ __attribute__((aligned(16))) unsigned short q_s[];   // [row_pad][kQStride]
    // kLds: [entry][row_pad] floats from byte plane_offset on (0 with one row tile: the queries then live in
    // registers once the loop starts), followed by the waves' [wave][2][row_pad] (reference, sum) pairs
    float* plane = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(q_s) + plane_offset);

    const unsigned task = blockIdx.z, h = blockIdx.y;
    const unsigned n_blocks = task_blocks(seg_off, seg_len, q_off, pruned_sel, task, max_blocks, tb);
    const unsigned S = n_blocks * kM;
    const unsigned chunk = kWaves * spans_per_wave * kSpan;
    const unsigned s_chunk = blockIdx.x * chunk;
    if (s_chunk >= S) { return; }
    const unsigned s_end = min(S, s_chunk + chunk);
    const unsigned s_last = s_end - 1;                   // last sub-block of this workgroup
    const unsigned g = q_heads / kv_heads, R = n_tokens * g;
    const int32_t psel = pruned_sel ? pruned_sel[task] : -1;
    const int32_t* pr = (pruned && psel >= 0) ? pruned + (static_cast<size_t>(psel) * kv_heads + h) * d_pruned : nullptr;

    // the wave index through readfirstlane: the compiler then knows that everything derived from it (a span's
    // position, whether a tile is cut by the task's end) is the same for all lanes and keeps it in scalar registers
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = lane >> 5, lr = lane & 31;
    const unsigned ksteps = d_pad / 16;                  // MFMA steps; lane half `half`, step ks takes piece 2*ks + half
    // the task's first representative: rows seg_off[task].. of the one table, or a table of the task's own
    const unsigned short* tbase =
        (task_tables ? static_cast<const unsigned short*>(task_tables[task]) + static_cast<int64_t>(h) * task_head_strides[task]
                     : table + static_cast<int64_t>(h) * head_stride + static_cast<int64_t>(seg_off[task]) * row_stride) +
        half * (8 * kM);

    // A span's keys: for each of its tiles, kSteps 16-byte loads per lane, piece 2*ks + half of the lane's
    // sub-block; the lanes of one instruction cover M*16 contiguous bytes per block and lane half.
    // Everything is unconditional - MFMA steps past d_pad reload piece 0 and are multiplied with a zero
    // query fragment, lanes and tiles past the workgroup's end reload its last vector and are masked or
    // never used.
    //
    // Three key buffers rotate, so two spans are in flight while one is worked on.  Every group of loads is
    // followed by a compiler barrier (an empty asm that may touch memory): left to itself the compiler sinks
    // a prefetch down to the span that consumes it - nothing but a loop exit lies between - and then nothing
    // is in flight.  The waits are the compiler's own: vector memory operations complete in issue order,
    // loads and stores alike, so it waits for "at most as many operations outstanding as were issued after
    // the loads of this span" - which only works because no store below is skipped on any path.
    auto load_keys = [&](u32x4 (&kf)[kLoads], unsigned s0) {
#pragma unroll
        for (int t = 0; t < kSpanTiles; ++t) {
            const unsigned s_mine = min(s0 + t * kTileSub + lr, s_last);
            const unsigned short* krow = tbase + static_cast<int64_t>(s_mine / kM) * row_stride + (s_mine % kM) * 8;
#pragma unroll
            for (int ks = 0; ks < kSteps; ++ks) {
                kf[t * kSteps + ks] = ucm::gload16(krow + (static_cast<unsigned>(ks) < ksteps ? ks : 0) * (16 * kM));
            }
        }
        asm volatile("" ::: "memory");
    };
    u32x4 k0[kLoads], k1[kLoads], k2[kLoads];
    const unsigned s_first = s_chunk + wave * kSpan;
    load_keys(k0, s_first);
    load_keys(k1, s_first + kStride);
    load_keys(k2, s_first + 2 * kStride);

    // ---- the head's query rows, gathered by the kept channels, zero padded (rows up to row_pad, columns up to 16*kSteps)
    constexpr unsigned kCols = 16 * kSteps;
    const unsigned short* qt = q + q_off[task];
    if (!pr && d_pruned == kCols && (d_orig % 8) == 0 && (reinterpret_cast<uintptr_t>(qt) & 15u) == 0) {
        constexpr unsigned cpr = kCols / 8;              // 16-byte pieces per row
        for (unsigned e = threadIdx.x; e < row_pad * cpr; e += kThreads) {
            const unsigned rho = e / cpr, c = e - rho * cpr;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (rho < R) {
                const unsigned xt = rho / g, gg = rho - xt * g;
                v = ucm::gload16(qt + (static_cast<size_t>(xt) * q_heads + h * g + gg) * d_orig + c * 8);
            }
            *reinterpret_cast<u32x4*>(&q_s[rho * kQStride + c * 8]) = v;
        }
    } else if (pr && q_full_ok && (reinterpret_cast<uintptr_t>(qt) & 15u) == 0) {
        // kept channels: whole query rows go to a second LDS area (coalesced, one round trip together with
        // the channel list) and are gathered from there
        unsigned short* q_full = q_s + row_pad * kQStride;
        const unsigned cpr = d_orig / 8;
        for (unsigned e = threadIdx.x; e < row_pad * cpr; e += kThreads) {
            const unsigned rho = e / cpr, c = e - rho * cpr;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (rho < R) {
                const unsigned xt = rho / g, gg = rho - xt * g;
                v = ucm::gload16(qt + (static_cast<size_t>(xt) * q_heads + h * g + gg) * d_orig + c * 8);
            }
            *reinterpret_cast<u32x4*>(&q_full[rho * kQStride + c * 8]) = v;
        }
        const unsigned p = threadIdx.x % kCols;          // kThreads is a multiple of kCols: a thread keeps its column
        const unsigned ch = p < d_pruned ? static_cast<unsigned>(pr[p]) : 0xffffffffu;
        __syncthreads();
        for (unsigned e = threadIdx.x; e < row_pad * kCols; e += kThreads) {
            const unsigned rho = e / kCols;
            q_s[rho * kQStride + p] = ch < d_orig ? q_full[rho * kQStride + ch] : static_cast<unsigned short>(0);
        }
    } else {
        for (unsigned e = threadIdx.x; e < row_pad * kCols; e += kThreads) {
            const unsigned rho = e / kCols, p = e - rho * kCols;
            unsigned short v = 0;
            if (rho < R && p < d_pruned) {
                const unsigned xt = rho / g, gg = rho - xt * g;
                const unsigned d = pr ? static_cast<unsigned>(pr[p]) : p;
                if (d < d_orig) { v = qt[(static_cast<size_t>(xt) * q_heads + h * g + gg) * d_orig + d]; }
            }
            q_s[rho * kQStride + p] = v;
        }
    }
    __syncthreads();

    // the query fragments do not change from tile to tile: with one row tile they stay in registers
    // (columns from d_pad to 16*kSteps are zero, so the reloaded key pieces of those steps do not count)
    u32x4 bq[kTwoRowTiles ? 1 : kSteps];
    if constexpr (!kTwoRowTiles) {
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
            bq[ks] = *reinterpret_cast<const u32x4*>(&q_s[lr * kQStride + half * 8 + ks * 16]);
        }
        if constexpr (kLds) { __syncthreads(); }         // every wave has its query fragments: the plane may overwrite them
    }

    float* wmax = ws_max + (static_cast<size_t>(task) * kv_heads + h) * (2 * row_pad) * max_tiles;          // [tile][2][row_pad]
    float* wpart = ws_part + (static_cast<size_t>(task) * kv_heads + h) * row_pad * kPartsPerTile * max_tiles;  // [part][row_pad]

    // Every exponential of a wave is taken relative to one reference per query row, the row's largest
    // score in the wave's first span, and not to the maximum of its own tile: fp32 has 2^127 of head room
    // above the reference, a term 2^126 below it may as well be zero, and the per-tile maxima (fifteen
    // v_max and a cross-lane move per sixteen scores), the rescaling of running sums and the exponentials
    // that go with it all disappear from the loop.  The negated reference is what the matrix cores start
    // accumulating from, so a score leaves them already shifted.  Should a span's sums ever pass 2^100
    // (a later score more than 69 above the reference), the reference is raised to that span's maximum,
    // the running sum is rescaled and the span is done again.
    float ref[kRowTiles], d_run[kRowTiles];              // ref: natural units; d_run: sum of exp(score - ref) so far
    f32x16 cinit[kRowTiles];
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt) {
        ref[rt] = -INFINITY;
        d_run[rt] = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) { cinit[rt][i] = 0.0f; }
    }
    auto query_fragment = [&](int rt, int ks) -> u32x4 {
        if constexpr (kTwoRowTiles) {
            return *reinterpret_cast<const u32x4*>(&q_s[(rt * 32 + lr) * kQStride + half * 8 + ks * 16]);
        } else {
            return bq[ks];
        }
    };
    // one tile's scores for row tile rt, added to what c holds
    auto tile_scores = [&](const u32x4 (&kf)[kLoads], int t, int rt, f32x16 c) -> f32x16 {
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kf[t * kSteps + ks]),
                                                       __builtin_bit_cast(f16x8, query_fragment(rt, ks)), c, 0, 0, 0);
        }
        return c;
    };
    // Lanes and tiles past the workgroup's end hold reloaded vectors of the task: they may take part.
    auto raise_ref = [&](const u32x4 (&kf)[kLoads]) {
#pragma unroll
        for (int rt = 0; rt < kRowTiles; ++rt) {
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < kSpanTiles; ++t) {
                f32x16 a;
#pragma unroll
                for (int i = 0; i < 16; ++i) { a[i] = 0.0f; }
                a = tile_scores(kf, t, rt, a);
#pragma unroll
                for (int i = 0; i < 16; ++i) { mx = fmaxf(mx, a[i]); }
            }
            const float nref = fmaxf(ref[rt], halves_max(mx));
            d_run[rt] *= __builtin_amdgcn_exp2f((ref[rt] - nref) * kLog2e);   // the first time: 0 * 2^-inf = 0
            ref[rt] = nref;
#pragma unroll
            for (int i = 0; i < 16; ++i) { cinit[rt][i] = -nref; }
        }
    };

    // One span: its sums go to the plane (or the workspace), their totals per row to span_total.
    auto span_sums = [&](const u32x4 (&kf)[kLoads], unsigned s_span, float (&span_total)[kRowTiles]) {
        {
            float e_sum[kRowTiles];                      // kLds, blocks longer than a tile: the plane entry being gathered
#pragma unroll
            for (int rt = 0; rt < kRowTiles; ++rt) { span_total[rt] = 0.0f; e_sum[rt] = 0.0f; }
#pragma unroll
            for (int t = 0; t < kSpanTiles; ++t) {
                const unsigned s0 = s_span + t * kTileSub;
                const unsigned tile = s0 / kTileSub;
                // a tile past the task's end is computed on reloaded keys, masked, and stored to padding
                const bool full = s0 + kTileSub <= S;    // wave-uniform; only a task's last tile needs the mask
                f32x16 acc[kRowTiles];
#pragma unroll
                for (int rt = 0; rt < kRowTiles; ++rt) { acc[rt] = tile_scores(kf, t, rt, cinit[rt]); }
#pragma unroll
                for (int rt = 0; rt < kRowTiles; ++rt) {
                    const unsigned rho = rt * 32 + lr;
                    float e[16];
#pragma unroll
                    for (int i = 0; i < 16; ++i) { e[i] = __builtin_amdgcn_exp2f(acc[rt][i] * kLog2e); }
                    if constexpr (kM < kTileSub) {
                        if (!full) {
                            // A task's last tile, or one past its end.  Rare and wave-uniform, so it has to stay
                            // a branch: turned into selects (with their compares hoisted to the head of the span)
                            // it costs more instructions per tile than the exponentials do.  What depends on a
                            // value that passed through an asm statement cannot be computed speculatively, which
                            // keeps the compiler from doing that.
                            unsigned left = s0 < S ? S - s0 : 0u;            // live sub-blocks of this tile
                            asm volatile("" : "+v"(left));
#pragma unroll
                            for (int i = 0; i < 16; ++i) {
                                e[i] = static_cast<unsigned>((i >> 2) * 8 + half * 4 + (i & 3)) < left ? e[i] : 0.0f;
                            }
                        }
                    }
                    // rows past R hold zero queries: they are computed like the rest and never read
                    const unsigned part0 = tile * kPartsPerTile;   // first part of the tile
                    // with 32 or more sub-blocks per block a tile is whole or past the task's end (its sums then go to
                    // padding and count as zero)
                    const bool dead = kM >= kTileSub && s0 >= S;
                    float total;
                    if constexpr (kLds) {
                        const float ref2 = ref[rt] * kLog2e;
                        if constexpr (kEntryTiles == 1) {
                            // an entry lies inside this tile: log2 of the block's sum of 2^(score*log2e)
                            total = block_sums<kTilePart>(e, half, [&](unsigned b, float v) {
                                plane[(part0 + b) * row_pad + rho] = ref2 + __builtin_amdgcn_logf(v);
                            });
                            total = dead ? 0.0f : total;
                        } else {
                            // an entry spans kEntryTiles tiles of this span
                            total = block_sums<kTilePart>(e, half, [](unsigned, float) {});
                            total = dead ? 0.0f : total;
                            e_sum[rt] = (t % kEntryTiles == 0) ? total : e_sum[rt] + total;
                            if (t % kEntryTiles == kEntryTiles - 1) {
                                plane[(tile / kEntryTiles) * row_pad + rho] = ref2 + __builtin_amdgcn_logf(e_sum[rt]);
                            }
                        }
                    } else {
                        total = block_sums<kTilePart>(e, half, [&](unsigned b, float v) {
                            wpart[static_cast<size_t>(part0 + b) * row_pad + rho] = v;
                        });
                        total = dead ? 0.0f : total;
                        // the pair the next kernel reads: what the tile's sums are relative to, and their total
                        wmax[(static_cast<size_t>(tile) * 2 + half) * row_pad + rho] = half ? total : ref[rt];
                    }
                    span_total[rt] += total;
                }
            }
        }
    };
    // At most two trips: the second only after the reference was raised.  The span's position passes through
    // an asm statement inside the loop: otherwise the compiler computes every store address of the span
    // ahead of the loop, which takes more registers than there are.
    auto process = [&](const u32x4 (&kf)[kLoads], unsigned s_span) {
#pragma unroll 1
        for (int pass = 0; pass < 2; ++pass) {
            unsigned s_here = s_span;
            asm volatile("" : "+s"(s_here));
            float span_total[kRowTiles];
            span_sums(kf, s_here, span_total);
            bool high = false;
#pragma unroll
            for (int rt = 0; rt < kRowTiles; ++rt) { high = high || span_total[rt] > 0x1p100f; }
            if (__builtin_expect(!__any(high), 1)) {
#pragma unroll
                for (int rt = 0; rt < kRowTiles; ++rt) { d_run[rt] += span_total[rt]; }
                break;
            }
            raise_ref(kf);                               // what this pass left in the plane is written again
        }
    };

    if (s_first < s_end) { raise_ref(k0); }

    for (unsigned s0 = s_first; s0 < s_end;) {
        process(k0, s0);
        load_keys(k0, s0 + 3 * kStride);
        s0 += kStride;
        if (s0 >= s_end) { break; }
        process(k1, s0);
        load_keys(k1, s0 + 3 * kStride);
        s0 += kStride;
        if (s0 >= s_end) { break; }
        process(k2, s0);
        load_keys(k2, s0 + 3 * kStride);
        s0 += kStride;
    }

    if constexpr (kLds) {
        // ---- this head's share of the votes, from the plane in LDS
        const unsigned plane_entries = kM < kTileSub ? max_tiles * kPartsPerTile : max_tiles / kEntryTiles;
        float* red = plane + static_cast<size_t>(plane_entries) * row_pad;   // [wave][2][row_pad]
        if (half == 0) {
#pragma unroll
            for (int rt = 0; rt < kRowTiles; ++rt) {
                red[(wave * 2 + 0) * row_pad + rt * 32 + lr] = ref[rt] * kLog2e;   // the same product the entries carry
                red[(wave * 2 + 1) * row_pad + rt * 32 + lr] = d_run[rt];
            }
        }
        __syncthreads();                                 // the plane and the waves' pairs are complete
        float row_m = 0.0f, row_w = 0.0f;
        if (threadIdx.x < row_pad) {
            row_m = red[threadIdx.x];                    // wave 0 always has a live tile, so its reference is finite
#pragma unroll
            for (int w = 1; w < kWaves; ++w) { row_m = fmaxf(row_m, red[(w * 2) * row_pad + threadIdx.x]); }
            float den = 0.0f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                den += red[(w * 2 + 1) * row_pad + threadIdx.x] * __builtin_amdgcn_exp2f(red[(w * 2) * row_pad + threadIdx.x] - row_m);
            }
            row_w = threadIdx.x < R ? 1.0f / den : 0.0f; // den is about 1 or more: the reference that became row_m is one of the row's scores; padding rows do not vote
        }
        __syncthreads();                                 // (a thread reads only its own column of the pairs)
        if (threadIdx.x < row_pad) {
            red[threadIdx.x] = row_m;
            red[row_pad + threadIdx.x] = row_w;
        }
        __syncthreads();
        // one thread per block walks the block's rows, starting at a row of its own so that the lanes of a
        // wave spread over the LDS banks
        float* vh = ws_part + (static_cast<size_t>(task) * kv_heads + h) * max_blocks;
        for (unsigned b = threadIdx.x; b < n_blocks; b += kThreads) {
            float v = 0.0f;
            for (unsigned entry = b * kEntriesPerBlock; entry < (b + 1) * kEntriesPerBlock; ++entry) {
                for (unsigned r = 0; r < row_pad; ++r) {
                    const unsigned rr = (r + b) & (row_pad - 1);
                    v += __builtin_amdgcn_exp2f(plane[entry * row_pad + rr] - red[rr]) * red[row_pad + rr];
                }
            }
            vh[b] = v;
        }
    }
}

// kLds path, grid: x = 256 blocks of the task, y = task: adds up the kv heads' shares of the votes.
__global__ __launch_bounds__(kThreads) void kvstar_headsum_kernel(
    const float* __restrict__ head_votes, const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len,
    const int64_t* __restrict__ q_off, const int32_t* __restrict__ pruned_sel, const TaskBounds tb,
    unsigned kv_heads, unsigned max_blocks, float* __restrict__ votes)
{
    const unsigned task = blockIdx.y, b = blockIdx.x * kThreads + threadIdx.x;
    if (b >= task_blocks(seg_off, seg_len, q_off, pruned_sel, task, max_blocks, tb)) { return; }
    float v = 0.0f;
    for (unsigned h = 0; h < kv_heads; ++h) { v += head_votes[(static_cast<size_t>(task) * kv_heads + h) * max_blocks + b]; }
    votes[seg_off[task] + b] = v;
}

// ---- votes: rescale to the row maximum, normalise, add the rows ---------------------------------------
// The workspace planes of a (task, kv head) keep the rows of one tile or block adjacent
// ([tile][2][row_pad], [block][row_pad]), so the score kernel's stores and the loads below move whole
// 128-byte lines.
//
// Phase 1, grid: x = kv head, y = task; thread = (group of tiles, row).  The tiles' (reference, sum) pairs
// give the row's largest reference - one of the row's scores, at most 2^100 below its largest - and the
// softmax denominator relative to it; each tile's reference in the workspace is replaced by the factor
// exp(tile reference - largest reference) / denominator the tile's partial sums have to be multiplied
// with.  Rows past tokens*group hold zero queries and are carried along.
__global__ __launch_bounds__(kThreads) void kvstar_rowscale_kernel(
    float* __restrict__ ws_max, const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len,
    const int64_t* __restrict__ q_off, const int32_t* __restrict__ pruned_sel, const TaskBounds tb, unsigned kv_heads,
    unsigned M, unsigned max_blocks, unsigned max_tiles, unsigned row_pad)
{
    __shared__ float red[kThreads];
    const unsigned task = blockIdx.y, h = blockIdx.x;
    const unsigned n_blocks = task_blocks(seg_off, seg_len, q_off, pruned_sel, task, max_blocks, tb);
    if (n_blocks == 0) { return; }
    const unsigned n_tiles = (n_blocks * M + kTileSub - 1) / kTileSub;
    const unsigned rho = threadIdx.x % row_pad, grp = threadIdx.x / row_pad, ngrp = kThreads / row_pad;
    float* tm = ws_max + (static_cast<size_t>(task) * kv_heads + h) * (2 * row_pad) * max_tiles + rho;   // [tile][2][row_pad]
    constexpr unsigned kMine = 16;                       // tiles a thread keeps in registers; the rest is re-read
    float mxs[kMine], sums[kMine];
    float mx = -INFINITY;
#pragma unroll
    for (unsigned u = 0; u < kMine; ++u) {
        const unsigned t = min(grp + u * ngrp, n_tiles - 1);   // clamped: unconditional loads, all in flight at once
        mxs[u] = tm[static_cast<size_t>(2 * t) * row_pad];
        sums[u] = tm[static_cast<size_t>(2 * t + 1) * row_pad];
    }
#pragma unroll
    for (unsigned u = 0; u < kMine; ++u) { mx = fmaxf(mx, mxs[u]); }
    for (unsigned t = grp + kMine * ngrp; t < n_tiles; t += ngrp) { mx = fmaxf(mx, tm[static_cast<size_t>(2 * t) * row_pad]); }
    red[threadIdx.x] = mx;
    __syncthreads();
    mx = red[rho];
    for (unsigned g = 1; g < ngrp; ++g) { mx = fmaxf(mx, red[g * row_pad + rho]); }
    __syncthreads();
    float den = 0.0f;
#pragma unroll
    for (unsigned u = 0; u < kMine; ++u) {
        if (grp + u * ngrp < n_tiles) { den += sums[u] * __expf(mxs[u] - mx); }
    }
    for (unsigned t = grp + kMine * ngrp; t < n_tiles; t += ngrp) {
        den += tm[static_cast<size_t>(2 * t + 1) * row_pad] * __expf(tm[static_cast<size_t>(2 * t) * row_pad] - mx);
    }
    red[threadIdx.x] = den;
    __syncthreads();
    den = red[rho];
    for (unsigned g = 1; g < ngrp; ++g) { den += red[g * row_pad + rho]; }
    const float inv = den > 1e-9f ? 1.0f / den : 1.0f;   // the reference skips the division then
#pragma unroll
    for (unsigned u = 0; u < kMine; ++u) {
        const unsigned t = grp + u * ngrp;
        if (t < n_tiles) { tm[static_cast<size_t>(2 * t) * row_pad] = __expf(mxs[u] - mx) * inv; }
    }
    for (unsigned t = grp + kMine * ngrp; t < n_tiles; t += ngrp) {
        tm[static_cast<size_t>(2 * t) * row_pad] = __expf(tm[static_cast<size_t>(2 * t) * row_pad] - mx) * inv;
    }
}

// Phase 2, grid: x = 8 blocks of the task, y = task; 32 lanes per block: votes[b] = sum over kv heads and
// rows of partial * factor.
__global__ __launch_bounds__(kThreads) void kvstar_vote_kernel(
    const float* __restrict__ ws_max, const float* __restrict__ ws_part, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, const int64_t* __restrict__ q_off, const int32_t* __restrict__ pruned_sel,
    const TaskBounds tb, unsigned R, unsigned kv_heads, unsigned M, unsigned max_blocks, unsigned max_tiles,
    unsigned row_pad, float* __restrict__ votes)
{
    constexpr unsigned kMaxHeads = 8;
    const unsigned task = blockIdx.y;
    const unsigned n_blocks = task_blocks(seg_off, seg_len, q_off, pruned_sel, task, max_blocks, tb);
    if (blockIdx.x * 8 >= n_blocks) { return; }
    const unsigned b = min(blockIdx.x * 8 + (threadIdx.x >> 5), n_blocks - 1), l32 = threadIdx.x & 31;
    const bool live = blockIdx.x * 8 + (threadIdx.x >> 5) < n_blocks;
    const unsigned part_sub = min(M, static_cast<unsigned>(kTileSub)), parts = M / part_sub;   // see kvstar_score_kernel
    const size_t plane_parts = static_cast<size_t>(max_tiles) * (kTileSub / part_sub);
    float v = 0.0f;
    for (unsigned part = b * parts; part < (b + 1) * parts; ++part) {
        const unsigned tile = (part * part_sub) / kTileSub;
        for (unsigned r0 = 0; r0 < R; r0 += 32) {
            const unsigned rho = min(r0 + l32, R - 1);   // clamped: every load is unconditional, the product is masked
            float p[kMaxHeads], f[kMaxHeads];
#pragma unroll
            for (unsigned h = 0; h < kMaxHeads; ++h) {
                const unsigned hh = min(h, kv_heads - 1);
                p[h] = ws_part[((static_cast<size_t>(task) * kv_heads + hh) * plane_parts + part) * row_pad + rho];
                f[h] = ws_max[((static_cast<size_t>(task) * kv_heads + hh) * max_tiles + tile) * (2 * row_pad) + rho];
            }
            if (r0 + l32 < R) {
#pragma unroll
                for (unsigned h = 0; h < kMaxHeads; ++h) { if (h < kv_heads) { v += p[h] * f[h]; } }
            }
        }
    }
#pragma unroll
    for (int d = 16; d >= 1; d >>= 1) { v += __shfl_xor(v, d, 64); }
    if (live && l32 == 0) { votes[seg_off[task] + b] = v; }
}

}  // namespace

// ---- query groups ----------------------------------------------------------------------------------
// The query tokens a step contributes to its requests' retrieval groups, copied aside as fp16: the reference clones
// one token per request and layer (save_to_standby, ucm/sparse/kvstar/multistep.py:318-324) and converts a group
// when it is retrieved (torch.stack(...).to(torch.float16), :252-254).  One workgroup per row; the conversion is
// the round-to-nearest-even one of that .to().
namespace {

template <int kType>   // UCM_DTYPE_*
__global__ __launch_bounds__(kThreads) void kvstar_park_kernel(
    const void* __restrict__ q, int64_t q_rows, unsigned row_elems, const int32_t* __restrict__ src_rows,
    const int64_t* __restrict__ dst_off, unsigned short* __restrict__ ring, int64_t ring_elems)
{
    const int64_t src = src_rows[blockIdx.x], dst = dst_off[blockIdx.x];
    // rows and places come from device memory: a row outside the queries or a place outside the ring is skipped
    if (src < 0 || src >= q_rows || dst < 0 || dst + row_elems > ring_elems || (dst & 7) != 0) { return; }
    unsigned short* out = ring + dst;
    for (unsigned e = threadIdx.x * 8; e < row_elems; e += kThreads * 8) {
        unsigned short h[8];
        if constexpr (kType == UCM_DTYPE_F16) {
            *reinterpret_cast<u32x4*>(h) = ucm::gload16(static_cast<const unsigned short*>(q) + src * row_elems + e);
        } else if constexpr (kType == UCM_DTYPE_BF16) {
            const u32x4 v = ucm::gload16(static_cast<const unsigned short*>(q) + src * row_elems + e);
            const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                h[2 * j] = f32_to_f16_bits(__uint_as_float(w[j] << 16));
                h[2 * j + 1] = f32_to_f16_bits(__uint_as_float(w[j] & 0xffff0000u));
            }
        } else {
            const float* f = static_cast<const float*>(q) + src * row_elems + e;
            const u32x4 a = ucm::gload16(f), b = ucm::gload16(f + 4);
            const unsigned w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) { h[j] = f32_to_f16_bits(__uint_as_float(w[j])); }
        }
        ucm::gstore16(out + e, *reinterpret_cast<const u32x4*>(h));
    }
}

}  // namespace

extern "C" int ucm_kvstar_park_queries(const void* q, int q_dtype, int64_t q_rows, int row_elems, const int32_t* src_rows,
                                       const int64_t* dst_off, int n, void* ring_f16, int64_t ring_elems, ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0 && q_rows >= 0 && ring_elems >= 0, "ucm_kvstar_park_queries: n=%d q_rows=%lld ring_elems=%lld", n,
                static_cast<long long>(q_rows), static_cast<long long>(ring_elems));
    if (n == 0) { return UCM_OK; }
    UCM_REQUIRE(q && src_rows && dst_off && ring_f16, "ucm_kvstar_park_queries: null pointer");
    UCM_REQUIRE(q_dtype == UCM_DTYPE_F32 || q_dtype == UCM_DTYPE_BF16 || q_dtype == UCM_DTYPE_F16, "ucm_kvstar_park_queries: q_dtype=%d", q_dtype);
    UCM_REQUIRE(row_elems > 0 && row_elems % 8 == 0, "ucm_kvstar_park_queries: row_elems=%d (a positive multiple of 8)", row_elems);
    UCM_REQUIRE(ucm::aligned16(q) && ucm::aligned16(ring_f16), "ucm_kvstar_park_queries: q and ring must be 16-byte aligned");
    UCM_REQUIRE(n <= 0x7fffffff, "ucm_kvstar_park_queries: n=%d", n);
    hipStream_t hs = ucm::as_stream(stream);
#define UCM_PARK(T)                                                                                                   \
    hipLaunchKernelGGL(kvstar_park_kernel<T>, dim3(static_cast<unsigned>(n)), dim3(kThreads), 0, hs, q, q_rows,       \
                       static_cast<unsigned>(row_elems), src_rows, dst_off, static_cast<unsigned short*>(ring_f16), ring_elems)
    if (q_dtype == UCM_DTYPE_F16) { UCM_PARK(UCM_DTYPE_F16); }
    else if (q_dtype == UCM_DTYPE_BF16) { UCM_PARK(UCM_DTYPE_BF16); }
    else { UCM_PARK(UCM_DTYPE_F32); }
#undef UCM_PARK
    UCM_LAUNCH_CHECK("ucm_kvstar_park_queries");
}

extern "C" int ucm_kvstar_block_repre_keys(const void* const* k_layers, int key_dtype, int n_layers, int num_blocks,
                                           const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                           int kv_heads, int head_dim, int merge, const int32_t* pruned,
                                           int64_t pruned_layer_stride, const int32_t* pruned_sel, int n_pruned_lists,
                                           int d_pruned, int d_pad, void* repre_f16, int repre_rows,
                                           int64_t repre_layer_stride, int64_t repre_head_stride, int64_t repre_row_stride,
                                           ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0, "ucm_kvstar_block_repre: n=%d", n);
    UCM_REQUIRE(key_dtype == UCM_DTYPE_BF16 || key_dtype == UCM_DTYPE_F16, "ucm_kvstar_block_repre: key_dtype=%d (bfloat16 or float16)",
                key_dtype);
    const bool f16 = key_dtype == UCM_DTYPE_F16;
    UCM_REQUIRE(!pruned_sel || (pruned && n_pruned_lists >= 1), "ucm_kvstar_block_repre: pruned_sel needs the lists and their number");
    const int lists_per_layer = pruned_sel ? n_pruned_lists : 1;
    if (n == 0) { return UCM_OK; }
    UCM_REQUIRE(k_layers && block_ids && slots && repre_f16, "ucm_kvstar_block_repre: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers <= 65535 && num_blocks > 0 && repre_rows > 0 && block_size > 0 && kv_heads > 0 &&
                    head_dim > 0, "ucm_kvstar_block_repre: non-positive shape");
    UCM_REQUIRE(merge > 0 && block_size % merge == 0, "ucm_kvstar_block_repre: merge=%d does not divide block_size=%d",
                merge, block_size);
    UCM_REQUIRE(d_pruned > 0 && d_pruned <= head_dim && d_pad >= d_pruned, "ucm_kvstar_block_repre: d_pruned=%d d_pad=%d",
                d_pruned, d_pad);
    UCM_REQUIRE(pruned || d_pruned == head_dim, "ucm_kvstar_block_repre: d_pruned < head_dim needs the channel list");
    UCM_REQUIRE(pruned_layer_stride == 0 || pruned_layer_stride >= static_cast<int64_t>(lists_per_layer) * kv_heads * d_pruned,
                "ucm_kvstar_block_repre: pruned_layer_stride=%lld", static_cast<long long>(pruned_layer_stride));
    const int M = block_size / merge;
    // a (row, kv head) cell is M*d_pad elements; the cells must not overlap: heads outside rows (head planes) or
    // rows outside heads (a block's heads next to each other)
    const int64_t cell = static_cast<int64_t>(M) * d_pad;
    UCM_REQUIRE(repre_row_stride >= cell && repre_head_stride >= cell &&
                    (repre_head_stride >= static_cast<int64_t>(repre_rows) * repre_row_stride ||
                     repre_row_stride >= static_cast<int64_t>(kv_heads) * repre_head_stride),
                "ucm_kvstar_block_repre: repre_head_stride=%lld and repre_row_stride=%lld let cells of %lld elements overlap",
                static_cast<long long>(repre_head_stride), static_cast<long long>(repre_row_stride),
                static_cast<long long>(cell));
    const unsigned row = static_cast<unsigned>(kv_heads) * static_cast<unsigned>(head_dim);
    UCM_SUPPORTED(row % 8 == 0 && d_pad % 8 == 0, "ucm_kvstar_block_repre: kv_heads*head_dim=%u and d_pad=%d must be multiples of 8",
                  row, d_pad);
    UCM_SUPPORTED(row <= 32768u && head_dim % 8 == 0, "ucm_kvstar_block_repre: kv_heads*head_dim=%u (at most 32768), head_dim=%d (a multiple of 8)", row, head_dim);
    const unsigned m_chunk = std::min<unsigned>(static_cast<unsigned>(M), 33280u / (row + 8));   // sub-blocks staged at a time: 65 KiB of LDS
    const size_t lds_bytes = static_cast<size_t>(m_chunk) * (row + 8) * 2 + (pruned ? static_cast<size_t>(kv_heads) * d_pruned * 4 : 0);
    UCM_REQUIRE(ucm::aligned16(repre_f16) && repre_layer_stride % 8 == 0 && repre_head_stride % 8 == 0 &&
                    repre_row_stride % 8 == 0, "ucm_kvstar_block_repre: table not 16-byte aligned");
    hipStream_t hs = ucm::as_stream(stream);
    // persistent workgroups for the common sub-block sizes: about 1024 over all layers (two fit a compute unit)
    const unsigned gx = static_cast<unsigned>(std::min(n, std::max(1, (1024 + n_layers - 1) / n_layers)));
#define UCM_KVSTAR_REPRE(MERGE)                                                                                        \
    do {                                                                                                             \
        if (f16) { UCM_KVSTAR_REPRE_T(MERGE, true); } else { UCM_KVSTAR_REPRE_T(MERGE, false); }                     \
    } while (0)
#define UCM_KVSTAR_REPRE_T(MERGE, F16)                                                                                 \
    do {                                                                                                             \
        if (lds_bytes > 48u * 1024u) {                                                                               \
            const hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(kvstar_repre_kernel<MERGE, F16>), \
                                                      hipFuncAttributeMaxDynamicSharedMemorySize,                   \
                                                      static_cast<int>(lds_bytes));                                \
            if (ea != hipSuccess) { return ucm::check_hip(ea, "ucm_kvstar_block_repre (LDS size)"); }                \
        }                                                                                                            \
        hipLaunchKernelGGL((kvstar_repre_kernel<MERGE, F16>), dim3(gx, n_layers), dim3(kThreads), lds_bytes, hs, k_layers,  \
                           block_ids, slots, static_cast<unsigned>(num_blocks), static_cast<unsigned>(n),            \
                           static_cast<unsigned>(repre_rows), static_cast<unsigned>(block_size),                     \
                           static_cast<unsigned>(kv_heads), static_cast<unsigned>(head_dim), pruned,                 \
                           pruned_layer_stride, pruned_sel, static_cast<unsigned>(lists_per_layer),                  \
                           static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad),                            \
                           static_cast<unsigned short*>(repre_f16), repre_layer_stride, repre_head_stride,          \
                           repre_row_stride, m_chunk);                                                               \
    } while (0)
    switch (merge) {
    case 1: UCM_KVSTAR_REPRE(1); break;
    case 2: UCM_KVSTAR_REPRE(2); break;
    case 4: UCM_KVSTAR_REPRE(4); break;
    case 8: UCM_KVSTAR_REPRE(8); break;
    default: {
        auto* any = f16 ? kvstar_repre_any_kernel<true> : kvstar_repre_any_kernel<false>;
        if (lds_bytes > 48u * 1024u) {
            const hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(any),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
            if (ea != hipSuccess) { return ucm::check_hip(ea, "ucm_kvstar_block_repre (LDS size)"); }
        }
        hipLaunchKernelGGL(any, dim3(static_cast<unsigned>(n), n_layers), dim3(kThreads), lds_bytes, hs,
                           k_layers, block_ids, slots, static_cast<unsigned>(num_blocks), static_cast<unsigned>(repre_rows),
                           static_cast<unsigned>(block_size), static_cast<unsigned>(kv_heads), static_cast<unsigned>(head_dim),
                           static_cast<unsigned>(merge), pruned, pruned_layer_stride, pruned_sel,
                           static_cast<unsigned>(lists_per_layer), static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad),
                           static_cast<unsigned short*>(repre_f16), repre_layer_stride, repre_head_stride, repre_row_stride,
                           m_chunk);
        break;
    }
    }
#undef UCM_KVSTAR_REPRE
#undef UCM_KVSTAR_REPRE_T
    UCM_LAUNCH_CHECK("ucm_kvstar_block_repre");
}

extern "C" int ucm_kvstar_block_repre(const void* const* k_layers, int n_layers, int num_blocks,
                                      const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                      int kv_heads, int head_dim, int merge, const int32_t* pruned,
                                      int64_t pruned_layer_stride, const int32_t* pruned_sel, int n_pruned_lists,
                                      int d_pruned, int d_pad, void* repre_f16, int repre_rows,
                                      int64_t repre_layer_stride, int64_t repre_head_stride, int64_t repre_row_stride,
                                      ucm_stream_t stream)
{
    return ucm_kvstar_block_repre_keys(k_layers, UCM_DTYPE_BF16, n_layers, num_blocks, block_ids, slots, n, block_size, kv_heads,
                                       head_dim, merge, pruned, pruned_layer_stride, pruned_sel, n_pruned_lists, d_pruned, d_pad,
                                       repre_f16, repre_rows, repre_layer_stride, repre_head_stride, repre_row_stride, stream);
}


namespace {
// Tiles the planes are sized for: a wave works in spans of up to four tiles and stores all of them
int64_t padded_tiles(int64_t sub_blocks_total)
{
    const int64_t tiles = (sub_blocks_total + kTileSub - 1) / kTileSub;
    return (tiles + 3) / 4 * 4;
}

// How one call is carried out: shared by the workspace sizing and the launch
struct VotePlan {
    unsigned max_tiles, row_pad, q_bytes, steps, span_tiles, plane_offset;
    size_t lds_plane;
    bool use_lds;
};

VotePlan plan_votes(int n_tasks, int kv_heads, int rows_per_head, int max_blocks, int sub_blocks, int d_pad, int tiles_per_wave)
{
    VotePlan p;
    p.max_tiles = static_cast<unsigned>(std::max<int64_t>(padded_tiles(static_cast<int64_t>(max_blocks) * sub_blocks), 4));
    p.row_pad = rows_per_head > 32 ? 64 : 32;
    p.q_bytes = p.row_pad * kQStride * 2;
    p.steps = d_pad <= 32 ? 2u : d_pad <= 64 ? 4u : 8u;        // MFMA steps per vector the kernel is built for
    p.span_tiles = 8u / p.steps;                               // tiles a wave moves at a time
    // One workgroup per (task, kv head) with the task's plane in LDS, when there are enough such workgroups to
    // fill the device and the plane fits; otherwise the workspace path, which may cut a task into chunks.
    // tiles_per_wave > 0 forces the workspace path, -1 the in-LDS path whenever the plane fits.
    p.plane_offset = rows_per_head > 32 ? p.q_bytes : 0u;
    const unsigned entry_tiles = static_cast<unsigned>(sub_blocks) <= kTileSub
                                     ? 1u : std::min<unsigned>(sub_blocks, p.span_tiles * kTileSub) / kTileSub;
    const size_t plane_entries = static_cast<unsigned>(sub_blocks) < kTileSub
                                     ? static_cast<size_t>(p.max_tiles) * (kTileSub / sub_blocks) : p.max_tiles / entry_tiles;
    p.lds_plane = p.plane_offset + plane_entries * p.row_pad * 4 + 2 * kWaves * p.row_pad * 4;
    p.use_lds = tiles_per_wave <= 0 && p.lds_plane <= kLdsPathMaxBytes &&
                (tiles_per_wave < 0 || static_cast<int64_t>(n_tasks) * kv_heads >= kLdsPathMinGroups);
    return p;
}
}  // namespace

namespace {
// floats a call carried out as `p` stores through ws_max / ws_part
void workspace_floats(const VotePlan& p, int n_tasks, int kv_heads, int max_blocks, int sub_blocks, int64_t* max_floats,
                      int64_t* part_floats)
{
    if (p.use_lds) {
        // only the kv heads' shares of the votes pass through memory
        *max_floats = 1;
        *part_floats = std::max<int64_t>(static_cast<int64_t>(n_tasks) * kv_heads * max_blocks, 1);
        return;
    }
    // per (task, kv head): a (reference, sum) pair per tile and row; a partial sum per row and block (per tile,
    // for blocks of more than 32 sub-blocks), padded to whole tiles
    const int64_t parts_per_tile = kTileSub / std::min(sub_blocks, kTileSub);
    *max_floats = static_cast<int64_t>(n_tasks) * kv_heads * p.row_pad * 2 * p.max_tiles;
    *part_floats = static_cast<int64_t>(n_tasks) * kv_heads * p.row_pad * parts_per_tile * p.max_tiles;
}
}  // namespace

extern "C" int ucm_kvstar_workspace_floats(int n_tasks, int kv_heads, int rows_per_head, int max_blocks, int sub_blocks,
                                           int d_pad, int tiles_per_wave, int64_t* max_floats, int64_t* part_floats)
{
    UCM_REQUIRE(tiles_per_wave >= -1, "ucm_kvstar_workspace_floats: tiles_per_wave=%d", tiles_per_wave);
    UCM_REQUIRE(n_tasks >= 0 && kv_heads > 0 && rows_per_head > 0 && rows_per_head <= kMaxRows && max_blocks >= 0 &&
                    sub_blocks > 0 && d_pad > 0 && max_floats && part_floats, "ucm_kvstar_workspace_floats: bad argument");
    UCM_REQUIRE(sub_blocks <= 128 && (sub_blocks & (sub_blocks - 1)) == 0, "ucm_kvstar_workspace_floats: sub_blocks=%d", sub_blocks);
    workspace_floats(plan_votes(n_tasks, kv_heads, rows_per_head, max_blocks, sub_blocks, d_pad, tiles_per_wave), n_tasks, kv_heads, max_blocks,
                     sub_blocks, max_floats, part_floats);
    return UCM_OK;
}

namespace {
int kvstar_votes(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads, int d_orig,
                 const int32_t* pruned, int n_lists, const int32_t* pruned_sel, int64_t rows_bound, const void* repre_f16, int64_t repre_head_stride, int64_t repre_row_stride,
                 const void* const* task_tables, const int64_t* task_head_strides, const int32_t* seg_off, const int32_t* seg_len, int n_tasks, int max_blocks,
                 int sub_blocks, int kv_heads, int d_pruned, int d_pad, float* ws_max, int64_t ws_max_floats, float* ws_part,
                 int64_t ws_part_floats, float* votes, int tiles_per_wave, ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks >= 0 && max_blocks >= 0, "ucm_kvstar_votes: n_tasks=%d max_blocks=%d", n_tasks, max_blocks);
    UCM_REQUIRE(q_elems >= 0 && rows_bound >= 0 && n_lists >= 0, "ucm_kvstar_votes: q_elems=%lld rows=%lld n_lists=%d",
                static_cast<long long>(q_elems), static_cast<long long>(rows_bound), n_lists);
    UCM_REQUIRE(tiles_per_wave >= -1, "ucm_kvstar_votes: tiles_per_wave=%d", tiles_per_wave);
    if (n_tasks == 0 || max_blocks == 0) { return UCM_OK; }
    UCM_REQUIRE(q_f16 && q_off && seg_off && seg_len && ws_max && ws_part && votes, "ucm_kvstar_votes: null pointer");
    UCM_REQUIRE(task_tables ? task_head_strides != nullptr : repre_f16 != nullptr, "ucm_kvstar_votes: no representative table");
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
    UCM_SUPPORTED(sub_blocks >= 1 && sub_blocks <= 128 && (sub_blocks & (sub_blocks - 1)) == 0,
                  "ucm_kvstar_votes: sub_blocks=%d (a power of two up to 128)", sub_blocks);
    UCM_REQUIRE(task_tables || (ucm::aligned16(repre_f16) && repre_head_stride % 8 == 0 && repre_head_stride > 0),
                "ucm_kvstar_votes: representatives not 16-byte aligned");
    UCM_REQUIRE(repre_row_stride % 8 == 0 && repre_row_stride >= static_cast<int64_t>(sub_blocks) * d_pad,
                "ucm_kvstar_votes: repre_row_stride=%lld (a multiple of 8, at least sub_blocks*d_pad=%d)",
                static_cast<long long>(repre_row_stride), sub_blocks * d_pad);
    const unsigned R = static_cast<unsigned>(n_tokens * (q_heads / kv_heads));
    const VotePlan plan = plan_votes(n_tasks, kv_heads, static_cast<int>(R), max_blocks, sub_blocks, d_pad, tiles_per_wave);
    {
        // the path depends on tiles_per_wave: a workspace sized for another value must not be overrun
        int64_t need_max = 0, need_part = 0;
        workspace_floats(plan, n_tasks, kv_heads, max_blocks, sub_blocks, &need_max, &need_part);
        UCM_REQUIRE(ws_max_floats >= need_max && ws_part_floats >= need_part,
                    "ucm_kvstar_votes: workspace of %lld + %lld floats, this call needs %lld + %lld (ucm_kvstar_workspace_floats)",
                    static_cast<long long>(ws_max_floats), static_cast<long long>(ws_part_floats),
                    static_cast<long long>(need_max), static_cast<long long>(need_part));
    }
    const unsigned max_tiles = plan.max_tiles, row_pad = plan.row_pad, q_bytes = plan.q_bytes, steps = plan.steps,
                   span_tiles = plan.span_tiles, plane_offset = plan.plane_offset;
    const size_t lds_plane = plan.lds_plane;
    const bool use_lds = plan.use_lds;
    // with channel lists, whole query rows are staged in a second area of q_bytes and gathered from there
    const unsigned q_full_ok = pruned != nullptr && d_orig % 8 == 0 && d_orig <= kMaxDim && ucm::aligned16(q_f16) ? 1u : 0u;
    const unsigned q_stage = q_full_ok ? 2 * q_bytes : q_bytes;
    const unsigned lds_bytes = use_lds ? static_cast<unsigned>(std::max<size_t>(lds_plane, q_stage)) : q_stage;
    // a workgroup stages its queries once, so it should walk many spans; the longest task is still cut into
    // enough chunks that about 2048 workgroups exist
    const unsigned max_spans = (max_tiles + span_tiles - 1) / span_tiles;
    const unsigned spans_per_wg_all = (max_spans + kWaves - 1) / kWaves;
    const unsigned want_chunks = use_lds ? 1u : std::max(1u, 2048u / static_cast<unsigned>(n_tasks * kv_heads));
    const unsigned spans_per_wave = tiles_per_wave > 0
                                        ? (static_cast<unsigned>(tiles_per_wave) + span_tiles - 1) / span_tiles
                                        : std::max(1u, (spans_per_wg_all + want_chunks - 1) / want_chunks);
    const unsigned chunks = (max_spans + kWaves * spans_per_wave - 1) / (kWaves * spans_per_wave);
    hipStream_t s = ucm::as_stream(stream);
    const TaskBounds tb = {rows_bound, q_elems, static_cast<int64_t>(n_tokens) * q_heads * d_orig, n_lists};
#define UCM_KVSTAR_ARGS dim3(chunks, kv_heads, n_tasks), dim3(kThreads), lds_bytes, s, static_cast<const unsigned short*>(q_f16), q_off, \
        static_cast<unsigned>(n_tokens), static_cast<unsigned>(q_heads), static_cast<unsigned>(d_orig), pruned, pruned_sel,   \
        static_cast<const unsigned short*>(repre_f16), task_tables, task_head_strides, seg_off, seg_len,                      \
        static_cast<unsigned>(kv_heads),                                                                                      \
        static_cast<unsigned>(d_pruned), static_cast<unsigned>(d_pad), repre_head_stride, repre_row_stride, ws_max, ws_part, \
        static_cast<unsigned>(max_blocks), max_tiles, spans_per_wave, row_pad, plane_offset, q_full_ok, tb
#define UCM_KVSTAR_LAUNCH4(M, STEPS, TWO, LDS)                                                                        \
    do {                                                                                                             \
        if (lds_bytes > 48u * 1024u) {                                                                               \
            const hipError_t ea = hipFuncSetAttribute(                                                               \
                reinterpret_cast<const void*>(kvstar_score_kernel<M, STEPS, TWO, LDS>),                              \
                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));                           \
            if (ea != hipSuccess) { return ucm::check_hip(ea, "ucm_kvstar_votes (LDS size)"); }                      \
        }                                                                                                            \
        hipLaunchKernelGGL((kvstar_score_kernel<M, STEPS, TWO, LDS>), UCM_KVSTAR_ARGS);                              \
    } while (0)
#define UCM_KVSTAR_LAUNCH3(M, STEPS, TWO)                                                                             \
    do {                                                                                                             \
        if (use_lds) { UCM_KVSTAR_LAUNCH4(M, STEPS, TWO, true); } else { UCM_KVSTAR_LAUNCH4(M, STEPS, TWO, false); } \
    } while (0)
#define UCM_KVSTAR_LAUNCH2(M, STEPS)                                                                                  \
    do {                                                                                                             \
        if (R > 32) { UCM_KVSTAR_LAUNCH3(M, STEPS, true); } else { UCM_KVSTAR_LAUNCH3(M, STEPS, false); }            \
    } while (0)
#define UCM_KVSTAR_LAUNCH(M)                                                                                          \
    do {                                                                                                             \
        if (steps == 2) { UCM_KVSTAR_LAUNCH2(M, 2); } else if (steps == 4) { UCM_KVSTAR_LAUNCH2(M, 4); }             \
        else { UCM_KVSTAR_LAUNCH2(M, 8); }                                                                           \
    } while (0)
    switch (sub_blocks) {
    case 1: UCM_KVSTAR_LAUNCH(1); break;
    case 2: UCM_KVSTAR_LAUNCH(2); break;
    case 4: UCM_KVSTAR_LAUNCH(4); break;
    case 8: UCM_KVSTAR_LAUNCH(8); break;
    case 16: UCM_KVSTAR_LAUNCH(16); break;
    case 32: UCM_KVSTAR_LAUNCH(32); break;
    case 64: UCM_KVSTAR_LAUNCH(64); break;
    default: UCM_KVSTAR_LAUNCH(128); break;
    }
#undef UCM_KVSTAR_LAUNCH
#undef UCM_KVSTAR_LAUNCH2
#undef UCM_KVSTAR_LAUNCH3
#undef UCM_KVSTAR_LAUNCH4
#undef UCM_KVSTAR_ARGS
    if (hipError_t e = hipGetLastError(); e != hipSuccess) { return ucm::check_hip(e, "ucm_kvstar_votes (scores)"); }
    if (use_lds) {
        hipLaunchKernelGGL(kvstar_headsum_kernel, dim3((max_blocks + kThreads - 1) / kThreads, n_tasks), dim3(kThreads), 0, s,
                           ws_part, seg_off, seg_len, q_off, pruned_sel, tb, static_cast<unsigned>(kv_heads),
                           static_cast<unsigned>(max_blocks), votes);
    } else {
        hipLaunchKernelGGL(kvstar_rowscale_kernel, dim3(static_cast<unsigned>(kv_heads), n_tasks), dim3(kThreads), 0, s, ws_max,
                           seg_off, seg_len, q_off, pruned_sel, tb, static_cast<unsigned>(kv_heads), static_cast<unsigned>(sub_blocks),
                           static_cast<unsigned>(max_blocks), max_tiles, row_pad);
        hipLaunchKernelGGL(kvstar_vote_kernel, dim3((max_blocks + 7) / 8, n_tasks), dim3(kThreads), 0, s, ws_max, ws_part,
                           seg_off, seg_len, q_off, pruned_sel, tb, R, static_cast<unsigned>(kv_heads),
                           static_cast<unsigned>(sub_blocks), static_cast<unsigned>(max_blocks), max_tiles, row_pad, votes);
    }
    UCM_LAUNCH_CHECK("ucm_kvstar_votes");
}
}  // namespace

extern "C" int ucm_kvstar_votes(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads,
                                int d_orig, const int32_t* pruned, int n_pruned_lists, const int32_t* pruned_sel,
                                const void* repre_f16, int64_t repre_rows, int64_t repre_head_stride,
                                int64_t repre_row_stride, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                                int max_blocks, int sub_blocks, int kv_heads, int d_pruned, int d_pad, float* ws_max,
                                int64_t ws_max_floats, float* ws_part, int64_t ws_part_floats, float* votes,
                                int tiles_per_wave, ucm_stream_t stream)
{
    return kvstar_votes(q_f16, q_elems, q_off, n_tokens, q_heads, d_orig, pruned, n_pruned_lists, pruned_sel, repre_rows, repre_f16,
                        repre_head_stride, repre_row_stride, nullptr, nullptr, seg_off, seg_len, n_tasks, max_blocks, sub_blocks,
                        kv_heads, d_pruned, d_pad, ws_max, ws_max_floats, ws_part, ws_part_floats, votes, tiles_per_wave, stream);
}

extern "C" int ucm_kvstar_votes_tables(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads,
                                       int d_orig, const int32_t* pruned, int n_pruned_lists, const int32_t* pruned_sel,
                                       const void* const* task_tables, const int64_t* task_head_strides,
                                       int64_t task_row_stride, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                                       int max_blocks, int sub_blocks, int kv_heads, int d_pruned, int d_pad, float* ws_max,
                                       int64_t ws_max_floats, float* ws_part, int64_t ws_part_floats, float* votes,
                                       int64_t votes_rows, int tiles_per_wave, ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks == 0 || (task_tables && task_head_strides), "ucm_kvstar_votes_tables: null table list");
    return kvstar_votes(q_f16, q_elems, q_off, n_tokens, q_heads, d_orig, pruned, n_pruned_lists, pruned_sel, votes_rows, nullptr, 0,
                        task_row_stride, task_tables, task_head_strides, seg_off, seg_len, n_tasks, max_blocks, sub_blocks,
                        kv_heads, d_pruned, d_pad, ws_max, ws_max_floats, ws_part, ws_part_floats, votes, tiles_per_wave, stream);
}
