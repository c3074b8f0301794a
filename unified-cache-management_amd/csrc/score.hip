// Query-vs-representative scores for a ragged batch, all layers in one launch.
//
// A single query per request makes this a GEMV: 2 flop per 4 bytes of
// representative, so the kernel is bounded by HBM and the matrix cores have
// nothing to contract.  What is fixed instead is the summation ORDER, which
// must reproduce the reference's AVX-512 dot product so that the block
// selection that follows is bit-identical:
//   * 16 lanes, lane j accumulating dims j, j+16, j+32, ... with one fma each;
//   * fold 16->8->4 (x[j] + x[j+8], then x[j] + x[j+4]), then (x0+x2)+(x1+x3);
//   * kv heads added in order starting from 0.0f.
// Mapping onto a 64-wide wavefront: four adjacent threads (a DPP quad) own one
// (block, head) vector; thread m of the quad holds AVX lanes 4m..4m+3 and reads
// one float4 per 16-dim step, so a wave streams 16 vectors = 8 KiB of
// contiguous representatives per pass with 16-byte loads, the two folds that
// cross threads are quad_perm DPP moves, and the last fold is in-register.
// The request's group-mean query is staged once per workgroup in LDS and then
// kept in registers (a thread's head never changes because kv_heads divides 16).
#include <algorithm>
#include <cfloat>

#include <cmath>

#include "common.h"
#include "topk_select.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxRow = 16 * 128;  // kv_heads * head_dim: what the staged query row may hold

template <int kCtrl>
__device__ __forceinline__ float quad_perm(float x)
{
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), kCtrl, 0xf, 0xf, true));
}
constexpr int kQuadXor2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kQuadXor1 = 0xB1;  // quad_perm:[1,0,3,2]

// four consecutive query elements, widened to fp32
__device__ __forceinline__ f32x4 load_q4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load_q4(const uint16_t* p)
{
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    f32x4 r = {__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
               __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u)};
    return r;
}

// fp16 queries travel as a type of their own so that the 16-bit loads pick the right widening
struct f16bits { uint16_t v; };
__device__ __forceinline__ f32x4 load_q4(const f16bits* p)
{
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 w = *reinterpret_cast<const h4*>(p);
    f32x4 r = {static_cast<float>(w.x), static_cast<float>(w.y), static_cast<float>(w.z), static_cast<float>(w.w)};
    return r;
}

// Group mean of four adjacent dims of one kv head: all kG loads are issued
// before the first add, the adds then run in head order (the reference's order).
template <int kG, typename QT>
__device__ __forceinline__ f32x4 group_mean4(const QT* src, int head_stride, float inv)
{
    f32x4 v[kG];
#pragma unroll
    for (int j = 0; j < kG; ++j) { v[j] = load_q4(src + j * head_stride); }
    f32x4 acc = v[0];
#pragma unroll
    for (int j = 1; j < kG; ++j) { acc = acc + v[j]; }
    return kG == 1 ? acc : acc * inv;
}

template <typename QT>
__device__ __forceinline__ f32x4 group_mean4_any(const QT* src, int head_stride, int g, float inv)
{
    switch (g) {
    case 1: return group_mean4<1>(src, head_stride, inv);
    case 2: return group_mean4<2>(src, head_stride, inv);
    case 4: return group_mean4<4>(src, head_stride, inv);
    case 8: return group_mean4<8>(src, head_stride, inv);
    default: break;
    }
    f32x4 acc = load_q4(src);
    for (int j = 1; j < g; ++j) { acc = acc + load_q4(src + j * head_stride); }
    return acc * inv;
}

// Plain loads on purpose: one instruction touches only 64 bytes (32 for the bf16
// table) of each 128-byte line and the next steps touch the rest, so the line
// has to stay in the vector L1 between them.  Nontemporal loads do not keep it
// there and every step then fetches the line from L2 again (bf16 table: 88 us
// instead of 47 us at 16 requests x 32 layers).
template <int kSteps>
__device__ __forceinline__ void load_pass(f32x4 (&kv)[kSteps], const float* p)
{
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        kv[i] = *reinterpret_cast<const f32x4*>(p + 16 * i);
    }
}

// One (block, head) dot product in the reference's order; all four threads of
// the quad return the same value.
template <int kSteps>
__device__ __forceinline__ float quad_dot(const f32x4 (&qr)[kSteps], const f32x4 (&kv)[kSteps])
{
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        a0 = __builtin_fmaf(qr[i].x, kv[i].x, a0);
        a1 = __builtin_fmaf(qr[i].y, kv[i].y, a1);
        a2 = __builtin_fmaf(qr[i].z, kv[i].z, a2);
        a3 = __builtin_fmaf(qr[i].w, kv[i].w, a3);
    }
    // lanes j and j+8 live two threads apart, j and j+4 one thread apart
    a0 = quad_perm<kQuadXor2>(a0) + a0; a1 = quad_perm<kQuadXor2>(a1) + a1;
    a2 = quad_perm<kQuadXor2>(a2) + a2; a3 = quad_perm<kQuadXor2>(a3) + a3;
    a0 = quad_perm<kQuadXor1>(a0) + a0; a1 = quad_perm<kQuadXor1>(a1) + a1;
    a2 = quad_perm<kQuadXor1>(a2) + a2; a3 = quad_perm<kQuadXor1>(a3) + a3;
    return (a0 + a2) + (a1 + a3);
}

// Finds the request that owns dense tile index `w` (tiles of all requests laid
// end to end, request r contributing ceil(seg_len[r] / tile_blocks) of them).
// Every wave does this on its own: 64 requests per trip, an inclusive wave scan
// of their tile counts, a ballot for the first prefix that exceeds w.
// A seg_len beyond the host's max_seg_len is cut there (the grid was sized for it); with min_tiles = 1 every
// request owns at least one tile, which the fused kernel needs: a request's last tile runs its selection.
__device__ __forceinline__ int clamped_len(int n, int max_seg_len) { return min(max(n, 0), max_seg_len); }

// The owner's other descriptors come back with it: every lane fetches its request's first row and query row together
// with its length, so the workgroup waits for memory once here, not once for the lengths and again for what they lead to.
__device__ __forceinline__ bool find_tile(const int32_t* __restrict__ seg_len, const int32_t* __restrict__ seg_off,
                                          const int32_t* __restrict__ q_rows, int n_req, int tile_blocks, int max_seg_len,
                                          int min_tiles, int w, int lane, int& r_out, int& tile_out, int& len_out,
                                          int& off_out, int& q_row_out)
{
    int base = 0;
    for (int c = 0; c < n_req; c += 64) {
        const int r = c + lane;
        const bool live = r < n_req;
        const int len = live ? clamped_len(seg_len[r], max_seg_len) : 0;
        const int off = live ? seg_off[r] : 0;
        const int qr = live && q_rows ? q_rows[r] : r;
        const int t = live ? max((len + tile_blocks - 1) / tile_blocks, min_tiles) : 0;
        int incl = t;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d, 64);
            if (lane >= d) { incl += up; }
        }
        const unsigned long long owner = __ballot(w < base + incl);
        if (owner) {
            const int src = __builtin_ctzll(owner);
            r_out = c + src;
            tile_out = w - (base + __shfl(incl - t, src, 64));
            len_out = __builtin_amdgcn_readlane(len, src);       // (scalar results: what follows stays uniform)
            off_out = __builtin_amdgcn_readlane(off, src);
            q_row_out = __builtin_amdgcn_readlane(qr, src);
            return true;
        }
        base += __shfl(incl, 63, 64);
    }
    return false;
}

// What a scoring launch reads and writes; the same for every workgroup.
struct ScoreArgs {
    const void* q;
    int64_t q_layer_stride;
    const int32_t* q_rows;
    int q_heads;
    const void* repre;
    int64_t repre_layer_stride;
    int64_t repre_rows;             // rows of a layer's table (and of a layer's scores): requests outside are skipped
    const int32_t* seg_off;
    const int32_t* seg_len;
    int n_req;
    int max_seg_len;
    int kv_heads;
    int num_repre;                  // representatives per (block, head): the score takes the largest of their dots
    float* scores;
    int64_t scores_layer_stride;
    int tile_blocks;
    float scale;
    int32_t* tickets;               // fused selection: [layers][n_req] counters, zero between launches; else null
};

// What a workgroup works on: request, tile, and whether the request's descriptors may be followed.
struct TileInfo {
    int r, tile, n;
    int64_t seg0, q_row;
    bool ok;
};

template <int kD>
__device__ __forceinline__ bool locate(const ScoreArgs& a, int lane, TileInfo& t)
{
    int len = 0, off = 0, q_row = 0;
    if (!find_tile(a.seg_len, a.seg_off, a.q_rows, a.n_req, a.tile_blocks, a.max_seg_len, a.tickets ? 1 : 0, blockIdx.y, lane,
                   t.r, t.tile, len, off, q_row)) {
        return false;
    }
    t.n = len;
    t.seg0 = off;
    // indices that came from device memory are followed only inside their tables: the request's query row
    // inside the layer's query block, its rows inside a layer of the representative table
    t.q_row = q_row;
    t.ok = !(a.q_rows && (t.q_row < 0 || (t.q_row + 1) * a.q_heads * kD > a.q_layer_stride)) &&
           t.seg0 >= 0 && t.seg0 + t.n <= a.repre_rows;
    return true;
}

// group-mean query -> LDS: sequential adds over the g heads of a group, then * (1/g)
template <int kD, typename QT>
__device__ __forceinline__ void stage_query(const ScoreArgs& a, int l, int64_t q_row, float* qbar)
{
    const int g = a.q_heads / a.kv_heads;
    const float inv = 1.0f / static_cast<float>(g);
    const QT* qp = static_cast<const QT*>(a.q) + static_cast<int64_t>(l) * a.q_layer_stride + q_row * a.q_heads * kD;
    for (int e = threadIdx.x * 4; e < a.kv_heads * kD; e += kThreads * 4) {
        const int hh = e / kD, d = e - hh * kD;
        const f32x4 mean = group_mean4_any(qp + static_cast<int64_t>(hh) * g * kD + d, kD, g, inv);
        *reinterpret_cast<f32x4*>(&qbar[e]) = mean;
    }
}

// Sum over the kv heads, in order, of the largest dot among a head's representatives
// (TopkBlockSelector::ComputeBlockScore); `first` is the lane that holds the block's first dot, `step` the lanes
// per vector.  With one representative per head this is s + fmaxf(-FLT_MAX, dot) per head.
__device__ __forceinline__ float head_sum(float dot, int first, int step, int kv_heads, int num_repre)
{
    float s = 0.0f;
    int src = first;
    for (int hh = 0; hh < kv_heads; ++hh) {
        float best = -FLT_MAX;
        for (int rr = 0; rr < num_repre; ++rr, src += step) { best = fmaxf(best, __shfl(dot, src, 64)); }
        s = s + best;
    }
    return s;
}

// A score on its way out.  With the selection fused in, another workgroup of this launch reads it: the store then
// goes through to memory at device scope (no cache of another part of the chip keeps it back), and the reader
// uses device-scope loads.
__device__ __forceinline__ void store_score(float* p, float v, bool through)
{
    if (through) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    else { *p = v; }
}

// The fused kernel's tail.  Every workgroup of a request takes a ticket once its scores have reached memory; the
// one that draws the last ticket resets the counter and its first wave runs the request's selection
// (TopkBlockSelector::TopKImpl, select_topk_block.cpp:20-51) on the scores all of them wrote.  Ordering: a wave's
// score stores are device-scope write-through stores, complete when the wave's memory counter reaches zero (the
// workgroup-scope fence below waits for that); the barrier then orders all waves' stores before thread 0's ticket;
// the last workgroup reads the scores with device-scope loads after it has seen every other ticket.  (A
// device-scope release/acquire pair would also do, but it writes the whole L2 back per wave: 7x the kernel's time.)
__device__ __forceinline__ void select_if_last(const ScoreArgs& a, const ucm::SelectArgs& sel, const TileInfo& t, int l)
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x >= 64) { return; }                           // the other waves are done: their registers are free again
    const int lane = threadIdx.x;
    int drawn = 0;
    int32_t* ticket = a.tickets + static_cast<int64_t>(l) * sel.cnt_layer_stride + t.r;
    if (lane == 0) { drawn = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    drawn = __builtin_amdgcn_readfirstlane(drawn);
    const int tiles = max((t.n + a.tile_blocks - 1) / a.tile_blocks, 1);
    if (drawn != tiles - 1) { return; }
    if (lane == 0) { __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    // the smallest tier of key registers that holds the request (the host allows at most 1024 blocks here)
    if (t.n <= 64) { ucm::select_wave<1, false, true>(sel, t.r, l, lane); }
    else if (t.n <= 128) { ucm::select_wave<2, false, true>(sel, t.r, l, lane); }
    else if (t.n <= 256) { ucm::select_wave<4, false, true>(sel, t.r, l, lane); }
    else if (t.n <= 512) { ucm::select_wave<8, false, true>(sel, t.r, l, lane); }
    else { ucm::select_wave<16, false, true>(sel, t.r, l, lane); }
}

// grid: x = layer, y = dense tile index over all requests (workgroups past the
// last tile exit).  Tiles are numbered densely and the layers run fastest, so that
// consecutive workgroups, which the hardware deals round-robin to the 8 XCDs,
// always carry work (with a (tile, request) grid the short requests of a ragged
// batch leave most XCDs idle) and the workgroups without a tile - the host sizes
// the grid from its own bounds on the segment lengths - are dispatched last: in
// between the others each of them held a workgroup's registers and LDS for the
// time it takes to find that out (12 us for 1600 of them among 2500).
template <int kD, typename QT>
__global__ __launch_bounds__(kThreads) void score_kernel(const ScoreArgs a, const ucm::SelectArgs sel)
{
    constexpr int kSteps = kD / 16;
    __shared__ __attribute__((aligned(16))) float qbar[kMaxRow];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l = blockIdx.x;
    const bool fused = a.tickets != nullptr;
    TileInfo t;
    if (!locate<kD>(a, lane, t)) { return; }
    const int tile0 = t.tile * a.tile_blocks;
    const int tile_end = min(tile0 + a.tile_blocks, t.n);
    if (t.ok && tile0 < tile_end) {                                  // (uniform over the workgroup)
        const int vecs = a.kv_heads * a.num_repre;  // vectors per block
        const int row = vecs * kD;

        const int m = lane & 3;                 // which 4 of the 16 lanes of the dot product
        const int v = lane >> 2;                // vector of this pass: 0..15
        const int blocks_per_pass = 16 / vecs;
        const int bl = v / vecs;                // block within the pass
        const int vb = v - bl * vecs;           // vector within the block, fixed for the whole kernel
        const int h = vb / a.num_repre;         // its kv head
        const int stride = kWaves * blocks_per_pass;

        const float* rbase = static_cast<const float*>(a.repre) + static_cast<int64_t>(l) * a.repre_layer_stride +
                             t.seg0 * row + vb * kD + 4 * m;
        float* sout = a.scores + static_cast<int64_t>(l) * a.scores_layer_stride + t.seg0;

        // the first pass's representatives are requested before the query is
        // touched, so the two latencies overlap
        int b0 = tile0 + wave * blocks_per_pass;
        f32x4 kv_a[kSteps], kv_b[kSteps];
        if (b0 < tile_end) { load_pass<kSteps>(kv_a, rbase + static_cast<int64_t>(min(b0 + bl, tile_end - 1)) * row); }

        stage_query<kD, QT>(a, l, t.q_row, qbar);
        __syncthreads();

        f32x4 qr[kSteps];
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
            qr[i] = *reinterpret_cast<const f32x4*>(&qbar[h * kD + 16 * i + 4 * m]);
        }

        // two passes per trip: the loads of the next pass are in flight while this one is reduced
        auto finish = [&](const f32x4 (&kv)[kSteps], int base) {
            const float dot = quad_dot<kSteps>(qr, kv);
            const float s = head_sum(dot, bl * vecs * 4, 4, a.kv_heads, a.num_repre);
            const int b = base + bl;
            if (b < tile_end && vb == 0 && m == 0) { store_score(sout + b, s * a.scale, fused); }   // (a scale of 1 changes no bit)
        };
        while (b0 < tile_end) {
            const int b1 = b0 + stride;
            if (b1 < tile_end) { load_pass<kSteps>(kv_b, rbase + static_cast<int64_t>(min(b1 + bl, tile_end - 1)) * row); }
            finish(kv_a, b0);
            if (b1 >= tile_end) { break; }
            const int b2 = b1 + stride;
            if (b2 < tile_end) { load_pass<kSteps>(kv_a, rbase + static_cast<int64_t>(min(b2 + bl, tile_end - 1)) * row); }
            finish(kv_b, b1);
            b0 = b2;
        }
    }
    if (fused) { select_if_last(a, sel, t, l); }
}

// ---- bf16 representative table ------------------------------------------------
// The live reference path stores block means rounded to the model dtype
// (ucm/sparse/gsa/gsa.py:640-652); keeping them as bf16 halves the bytes this
// kernel streams and widens to the same fp32 values.  Two adjacent threads own
// one (block, head) vector: thread p holds AVX lanes 8p..8p+7 and reads eight
// bf16 (16 bytes) per 16-dim step, a wave covers 32 vectors = 8 KiB per pass;
// the j/j+8 fold crosses the pair (one DPP), the j/j+4 and final folds are
// in-register.  Same arithmetic, same order, same bits as the fp32-table kernel.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int kSteps>
__device__ __forceinline__ void load_pass_bf16(u32x4 (&kv)[kSteps], const uint16_t* p)
{
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        kv[i] = *reinterpret_cast<const u32x4*>(p + 16 * i);
    }
}

template <int kSteps>
__device__ __forceinline__ float pair_dot(const f32x4 (&qlo)[kSteps], const f32x4 (&qhi)[kSteps],
                                          const u32x4 (&kv)[kSteps])
{
    float a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        a[0] = __builtin_fmaf(qlo[i].x, __uint_as_float(kv[i].x << 16), a[0]);
        a[1] = __builtin_fmaf(qlo[i].y, __uint_as_float(kv[i].x & 0xffff0000u), a[1]);
        a[2] = __builtin_fmaf(qlo[i].z, __uint_as_float(kv[i].y << 16), a[2]);
        a[3] = __builtin_fmaf(qlo[i].w, __uint_as_float(kv[i].y & 0xffff0000u), a[3]);
        a[4] = __builtin_fmaf(qhi[i].x, __uint_as_float(kv[i].z << 16), a[4]);
        a[5] = __builtin_fmaf(qhi[i].y, __uint_as_float(kv[i].z & 0xffff0000u), a[5]);
        a[6] = __builtin_fmaf(qhi[i].z, __uint_as_float(kv[i].w << 16), a[6]);
        a[7] = __builtin_fmaf(qhi[i].w, __uint_as_float(kv[i].w & 0xffff0000u), a[7]);
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) { a[c] = quad_perm<kQuadXor1>(a[c]) + a[c]; }   // lanes j and j+8: the other thread
    const float b0 = a[4] + a[0], b1 = a[5] + a[1], b2 = a[6] + a[2], b3 = a[7] + a[3];   // j and j+4
    return (b0 + b2) + (b1 + b3);
}

template <int kD, typename QT>
__global__ __launch_bounds__(kThreads) void score_kernel_bf16(const ScoreArgs a, const ucm::SelectArgs sel)
{
    constexpr int kSteps = kD / 16;
    __shared__ __attribute__((aligned(16))) float qbar[kMaxRow];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l = blockIdx.x;
    const bool fused = a.tickets != nullptr;
    TileInfo t;
    if (!locate<kD>(a, lane, t)) { return; }
    const int tile0 = t.tile * a.tile_blocks;
    const int tile_end = min(tile0 + a.tile_blocks, t.n);
    if (t.ok && tile0 < tile_end) {                                  // (uniform over the workgroup)
        const int vecs = a.kv_heads * a.num_repre;
        const int row = vecs * kD;

        const int p = lane & 1;                 // which 8 of the 16 lanes of the dot product
        const int v = lane >> 1;                // vector of this pass: 0..31
        const int blocks_per_pass = 32 / vecs;
        const int bl = v / vecs;
        const int vb = v - bl * vecs;
        const int h = vb / a.num_repre;
        const int stride = kWaves * blocks_per_pass;

        const uint16_t* rbase = static_cast<const uint16_t*>(a.repre) + static_cast<int64_t>(l) * a.repre_layer_stride +
                                t.seg0 * row + vb * kD + 8 * p;
        float* sout = a.scores + static_cast<int64_t>(l) * a.scores_layer_stride + t.seg0;

        // Loads and the store below are unconditional (rows and the output index are clamped to the tile's last
        // block, whose score is then written more than once): an operation skipped on some path would make the
        // compiler wait for everything outstanding, the prefetch included.  The empty asm keeps the compiler from
        // sinking a prefetch down to its use.
        int b0 = tile0 + wave * blocks_per_pass;
        u32x4 kv_a[kSteps], kv_b[kSteps];
        load_pass_bf16<kSteps>(kv_a, rbase + static_cast<int64_t>(min(b0 + bl, tile_end - 1)) * row);
        asm volatile("" ::: "memory");

        stage_query<kD, QT>(a, l, t.q_row, qbar);
        __syncthreads();

        // Half of the thread's query values stay in registers, the other half is read from LDS again in every pass
        // (broadcast reads, after the memory clobber that follows the prefetch): with all of them in registers the
        // kernel needs 158 VGPRs and runs three waves per SIMD, with half it needs 126 and runs four, which is worth
        // 8 % on long requests (80 layers x 8 requests x 523-981 blocks: 239 -> 220 us) and costs the ragged batch
        // of 16 short requests nothing; all of them from LDS (97 VGPRs, still four waves) was 211 us there but 56
        // instead of 51 us on the ragged batch, whose workgroups make only a few passes.
        const float* qmine = &qbar[h * kD + 8 * p];
        f32x4 ql[kSteps];
#pragma unroll
        for (int i = 0; i < kSteps; ++i) { ql[i] = *reinterpret_cast<const f32x4*>(qmine + 16 * i); }
        auto finish = [&](const u32x4 (&kv)[kSteps], int base) {
            f32x4 qh[kSteps];
#pragma unroll
            for (int i = 0; i < kSteps; ++i) { qh[i] = *reinterpret_cast<const f32x4*>(qmine + 16 * i + 4); }
            const float dot = pair_dot<kSteps>(ql, qh, kv);
            const float s = head_sum(dot, bl * vecs * 2, 2, a.kv_heads, a.num_repre);
            // the lanes of a block all hold its score; a scale of 1 changes no bit
            store_score(sout + min(base + bl, tile_end - 1), s * a.scale, fused);
        };
        while (b0 < tile_end) {
            const int b1 = b0 + stride;
            load_pass_bf16<kSteps>(kv_b, rbase + static_cast<int64_t>(min(b1 + bl, tile_end - 1)) * row);
            asm volatile("" ::: "memory");
            finish(kv_a, b0);
            if (b1 >= tile_end) { break; }
            const int b2 = b1 + stride;
            load_pass_bf16<kSteps>(kv_a, rbase + static_cast<int64_t>(min(b2 + bl, tile_end - 1)) * row);
            asm volatile("" ::: "memory");
            finish(kv_b, b1);
            b0 = b2;
        }
    }
    if (fused) { select_if_last(a, sel, t, l); }
}

template <int kD, typename QT>
void launch_dim(const ScoreArgs& a, const ucm::SelectArgs& sel, bool bf16_table, dim3 grid, hipStream_t s)
{
    if (bf16_table) { hipLaunchKernelGGL((score_kernel_bf16<kD, QT>), grid, dim3(kThreads), 0, s, a, sel); }
    else { hipLaunchKernelGGL((score_kernel<kD, QT>), grid, dim3(kThreads), 0, s, a, sel); }
}

template <int kD>
void launch_q(const ScoreArgs& a, const ucm::SelectArgs& sel, int q_dtype, bool bf16_table, dim3 grid, hipStream_t s)
{
    if (q_dtype == UCM_DTYPE_F32) { launch_dim<kD, float>(a, sel, bf16_table, grid, s); }
    else if (q_dtype == UCM_DTYPE_BF16) { launch_dim<kD, uint16_t>(a, sel, bf16_table, grid, s); }
    else { launch_dim<kD, f16bits>(a, sel, bf16_table, grid, s); }
}

// Host checks shared by ucm_score_blocks and ucm_score_select, then the launch.  `sel` is null for scores alone.
int score_launch(const char* name, const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows, int q_heads,
                 const void* repre, int repre_dtype, int64_t repre_layer_stride, int64_t repre_rows, int num_repre,
                 const int32_t* seg_off, const int32_t* seg_len, int n_req, int max_seg_len, int64_t total_blocks,
                 int n_layers, int kv_heads, int head_dim, float* scores, int64_t scores_layer_stride, float scale,
                 int tile_blocks_arg, const ucm::SelectArgs* sel, int32_t* tickets, ucm_stream_t stream)
{
    UCM_REQUIRE(std::isfinite(scale), "%s: scale is not finite", name);
    UCM_REQUIRE(tile_blocks_arg >= 0 && tile_blocks_arg <= 4096, "%s: tile_blocks=%d", name, tile_blocks_arg);
    UCM_REQUIRE(n_req == 0 || max_seg_len == 0 || (q && repre && seg_off && seg_len && scores), "%s: null pointer", name);
    UCM_REQUIRE(q_dtype == UCM_DTYPE_F32 || q_dtype == UCM_DTYPE_BF16 || q_dtype == UCM_DTYPE_F16, "%s: q_dtype=%d", name, q_dtype);
    UCM_REQUIRE(repre_dtype == UCM_DTYPE_F32 || repre_dtype == UCM_DTYPE_BF16, "%s: repre_dtype=%d", name, repre_dtype);
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535, "%s: n_req=%d n_layers=%d", name, n_req, n_layers);
    UCM_REQUIRE(max_seg_len >= 0 && total_blocks >= 0, "%s: max_seg_len=%d total_blocks=%lld", name, max_seg_len,
                static_cast<long long>(total_blocks));
    UCM_REQUIRE(kv_heads > 0 && q_heads >= kv_heads && q_heads % kv_heads == 0, "%s: q_heads=%d kv_heads=%d", name, q_heads, kv_heads);
    UCM_REQUIRE(num_repre >= 1, "%s: num_repre=%d", name, num_repre);
    UCM_SUPPORTED(head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128 || head_dim == 192 || head_dim == 256,
                  "%s: head_dim=%d (32, 64, 96, 128, 192 or 256)", name, head_dim);
    const int vecs = kv_heads * num_repre;
    UCM_SUPPORTED(vecs * head_dim <= kMaxRow, "%s: kv_heads*num_repre*head_dim=%d (at most %d)", name, vecs * head_dim, kMaxRow);
    UCM_SUPPORTED(vecs <= 16 && 16 % vecs == 0, "%s: kv_heads*num_repre=%d (1, 2, 4, 8 or 16)", name, vecs);
    const int es = repre_dtype == UCM_DTYPE_BF16 ? 2 : 4;
    UCM_REQUIRE(ucm::aligned16(repre) && repre_layer_stride % (16 / es) == 0, "%s: repre not 16-byte aligned", name);
    UCM_REQUIRE(ucm::aligned16(q) && q_layer_stride % 8 == 0, "%s: q not 16-byte aligned", name);
    UCM_REQUIRE(!q_rows || q_layer_stride >= static_cast<int64_t>(q_heads) * head_dim,
                "%s: with q_rows, q_layer_stride=%lld bounds the rows and must hold at least one", name,
                static_cast<long long>(q_layer_stride));
    UCM_REQUIRE(repre_rows >= 0 && (n_layers == 1 || (repre_layer_stride >= repre_rows * vecs * head_dim &&
                                                     scores_layer_stride >= repre_rows)),
                "%s: repre_rows=%lld does not fit the layer strides", name, static_cast<long long>(repre_rows));
    if (n_req == 0 || (max_seg_len == 0 && !sel)) { return UCM_OK; }
    // upper bound of sum(ceil(seg_len / tile)): exact to within n_req when the host knows the total
    const int row_bytes = vecs * head_dim * es;
    int tile_blocks = tile_blocks_arg > 0 ? tile_blocks_arg : std::max(8, (128 * 1024) / row_bytes);
    if (tile_blocks_arg <= 0) {
        // a launch over one layer or few short requests: smaller tiles until about half the chip's CUs have a
        // workgroup (one layer of 16 requests x 240 blocks: 16.0 us with 77 workgroups, 14.2 us with 137)
        const int64_t blocks = total_blocks > 0 ? total_blocks : static_cast<int64_t>(max_seg_len) * n_req;
        while (tile_blocks > 16 && (blocks / tile_blocks + n_req) * n_layers < 128) { tile_blocks /= 2; }
    }
    const int64_t per_req = std::max<int64_t>((static_cast<int64_t>(max_seg_len) + tile_blocks - 1) / tile_blocks, sel ? 1 : 0);
    int64_t tile_bound = per_req * n_req;
    // (with the selection fused in, every tile of every request has to run, whatever seg_len holds: the
    // caller's total is not used to shrink the grid)
    if (total_blocks > 0 && !sel) { tile_bound = std::min(tile_bound, (total_blocks + tile_blocks - 1) / tile_blocks + n_req); }
    UCM_REQUIRE(tile_bound <= 65535, "%s: too many tiles for one launch (%lld)", name, static_cast<long long>(tile_bound));
    const ScoreArgs a = {q, q_layer_stride, q_rows, q_heads, repre, repre_layer_stride, repre_rows, seg_off, seg_len, n_req,
                         max_seg_len, kv_heads, num_repre, scores, scores_layer_stride, tile_blocks, scale, sel ? tickets : nullptr};
    const ucm::SelectArgs none = {};
    const dim3 grid(n_layers, static_cast<unsigned>(tile_bound));
    hipStream_t s = ucm::as_stream(stream);
    const bool bf16_table = repre_dtype == UCM_DTYPE_BF16;
    switch (head_dim) {
    case 32: launch_q<32>(a, sel ? *sel : none, q_dtype, bf16_table, grid, s); break;
    case 64: launch_q<64>(a, sel ? *sel : none, q_dtype, bf16_table, grid, s); break;
    case 96: launch_q<96>(a, sel ? *sel : none, q_dtype, bf16_table, grid, s); break;
    case 128: launch_q<128>(a, sel ? *sel : none, q_dtype, bf16_table, grid, s); break;
    case 192: launch_q<192>(a, sel ? *sel : none, q_dtype, bf16_table, grid, s); break;
    default: launch_q<256>(a, sel ? *sel : none, q_dtype, bf16_table, grid, s); break;
    }
    return ucm::check_hip(hipGetLastError(), name);
}

}  // namespace

extern "C" int ucm_score_blocks(const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows,
                                int q_heads, const void* repre, int repre_dtype, int64_t repre_layer_stride,
                                int64_t repre_rows, int num_repre, const int32_t* seg_off, const int32_t* seg_len,
                                int n_req, int max_seg_len, int64_t total_blocks, int n_layers, int kv_heads,
                                int head_dim, float* scores, int64_t scores_layer_stride, float scale,
                                int tile_blocks, ucm_stream_t stream)
{
    return score_launch("ucm_score_blocks", q, q_dtype, q_layer_stride, q_rows, q_heads, repre, repre_dtype, repre_layer_stride,
                        repre_rows, num_repre, seg_off, seg_len, n_req, max_seg_len, total_blocks, n_layers, kv_heads, head_dim,
                        scores, scores_layer_stride, scale, tile_blocks, nullptr, nullptr, stream);
}

extern "C" int ucm_score_select(const ucm_score_select_args_t* p, ucm_stream_t stream)
{
    UCM_REQUIRE(p && p->struct_size == sizeof(ucm_score_select_args_t), "ucm_score_select: args missing or of another version (struct_size)");
    const int n_req = p->n_req, n_layers = p->n_layers, first = p->first_layer;
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535 && first >= 0, "ucm_score_select: n_req=%d n_layers=%d first_layer=%d",
                n_req, n_layers, first);
    if (n_req == 0) { return UCM_OK; }
    UCM_REQUIRE(p->seg_off && p->seg_len && p->topk_len && p->idx_out && p->count_out && p->tickets && p->scores,
                "ucm_score_select: null pointer");
    UCM_REQUIRE(p->start_w >= 0 && p->end_w >= 0 && p->max_seg_len >= 0, "ucm_score_select: negative window or length");
    UCM_REQUIRE(p->out_stride >= p->max_seg_len, "ucm_score_select: out_stride=%d < max_seg_len=%d", p->out_stride, p->max_seg_len);
    UCM_REQUIRE((p->block_tables == nullptr) == (p->phys_out == nullptr), "ucm_score_select: block_tables and phys_out go together");
    UCM_REQUIRE(!p->block_tables || p->bt_stride >= p->max_seg_len, "ucm_score_select: bt_stride=%d < max_seg_len=%d", p->bt_stride,
                p->max_seg_len);
    UCM_REQUIRE(!p->sparse_seq_lens || (p->seq_lens && p->block_size > 0), "ucm_score_select: sparse_seq_lens needs seq_lens and block_size");
    UCM_SUPPORTED(p->max_seg_len <= 1024, "ucm_score_select: max_seg_len=%d (at most 1024 blocks per request; ucm_score_blocks + "
                  "ucm_topk_windows take up to 4096)", p->max_seg_len);
    UCM_REQUIRE(p->kv_heads > 0 && p->head_dim > 0 && p->num_repre >= 1, "ucm_score_select: kv_heads=%d head_dim=%d num_repre=%d",
                p->kv_heads, p->head_dim, p->num_repre);
    // table pointers name layer 0 and move to first_layer here; q names the first layer scored
    const int64_t es = p->repre_dtype == UCM_DTYPE_BF16 ? 2 : 4;
    const char* repre = static_cast<const char*>(p->repre) + first * p->repre_layer_stride * es;
    float* scores = p->scores + first * p->scores_layer_stride;
    UCM_REQUIRE(p->idx_layer_stride >= 0 && p->count_layer_stride >= 0, "ucm_score_select: negative layer stride");
    const int64_t idx_ls = p->idx_layer_stride ? p->idx_layer_stride : static_cast<int64_t>(n_req) * p->out_stride;
    const int64_t cnt_ls = p->count_layer_stride ? p->count_layer_stride : n_req;
    UCM_REQUIRE(idx_ls >= static_cast<int64_t>(n_req) * p->out_stride && cnt_ls >= n_req,
                "ucm_score_select: layer strides shorter than a layer (%lld, %lld)", static_cast<long long>(idx_ls),
                static_cast<long long>(cnt_ls));
    const ucm::SelectArgs sel = {scores, p->scores_layer_stride, p->repre_rows, p->seg_off, p->seg_len, p->topk_len, n_req,
                                 p->max_seg_len, p->start_w, p->end_w, p->idx_out + first * idx_ls, p->out_stride, idx_ls, cnt_ls,
                                 p->count_out + first * cnt_ls, p->block_tables, p->bt_stride,
                                 p->phys_out ? p->phys_out + first * idx_ls : nullptr, p->seq_lens, p->block_size,
                                 p->sparse_seq_lens ? p->sparse_seq_lens + first * cnt_ls : nullptr};
    return score_launch("ucm_score_select", p->q, p->q_dtype, p->q_layer_stride, p->q_rows, p->q_heads, repre, p->repre_dtype,
                        p->repre_layer_stride, p->repre_rows, p->num_repre, p->seg_off, p->seg_len, n_req, p->max_seg_len,
                        p->total_blocks,
                        n_layers, p->kv_heads, p->head_dim, scores, p->scores_layer_stride, p->scale, p->tile_blocks, &sel,
                        p->tickets + first * cnt_ls, stream);
}
