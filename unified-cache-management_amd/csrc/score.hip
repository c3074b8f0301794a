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
__device__ __forceinline__ bool find_tile(const int32_t* __restrict__ seg_len, int n_req, int tile_blocks,
                                          int w, int lane, int& r_out, int& tile_out)
{
    int base = 0;
    for (int c = 0; c < n_req; c += 64) {
        const int r = c + lane;
        const int t = r < n_req ? (max(seg_len[r], 0) + tile_blocks - 1) / tile_blocks : 0;
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
            return true;
        }
        base += __shfl(incl, 63, 64);
    }
    return false;
}

// grid: x = dense tile index over all requests (workgroups past the last tile
// exit), y = layer.  Tiles are numbered densely so that consecutive workgroups,
// which the hardware deals round-robin to the 8 XCDs, always carry work: with a
// (tile, request) grid the short requests of a ragged batch leave most XCDs idle.
template <int kD, typename QT>
__global__ __launch_bounds__(kThreads) void score_kernel(
    const QT* __restrict__ q, int64_t q_layer_stride, const int32_t* __restrict__ q_rows, int q_heads,
    const float* __restrict__ repre, int64_t repre_layer_stride, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, int n_req, int kv_heads, float* __restrict__ scores,
    int64_t scores_layer_stride, int tile_blocks, float scale)
{
    constexpr int kSteps = kD / 16;
    __shared__ __attribute__((aligned(16))) float qbar[kMaxRow];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l = blockIdx.y;
    int r, tile;
    if (!find_tile(seg_len, n_req, tile_blocks, blockIdx.x, lane, r, tile)) { return; }
    // a row index that came from device memory is followed only inside the layer's query block
    const int64_t q_row = q_rows ? static_cast<int64_t>(q_rows[r]) : r;
    if (q_rows && (q_row < 0 || (q_row + 1) * q_heads * kD > q_layer_stride)) { return; }   // (the whole workgroup)
    const int n = seg_len[r];
    const int tile0 = tile * tile_blocks;
    const int tile_end = min(tile0 + tile_blocks, n);
    const int row = kv_heads * kD;

    const int m = lane & 3;                 // which 4 of the 16 lanes of the dot product
    const int v = lane >> 2;                // vector of this pass: 0..15
    const int blocks_per_pass = 16 / kv_heads;
    const int bl = v / kv_heads;            // block within the pass
    const int h = v - bl * kv_heads;        // kv head, fixed for the whole kernel
    const int stride = kWaves * blocks_per_pass;
    const int seg0 = seg_off[r];

    const float* rbase = repre + static_cast<int64_t>(l) * repre_layer_stride +
                         static_cast<int64_t>(seg0) * row + h * kD + 4 * m;
    float* sout = scores + static_cast<int64_t>(l) * scores_layer_stride + seg0;

    // the first pass's representatives are requested before the query is
    // touched, so the two latencies overlap
    int b0 = tile0 + wave * blocks_per_pass;
    f32x4 kv_a[kSteps], kv_b[kSteps];
    if (b0 < tile_end) { load_pass<kSteps>(kv_a, rbase + static_cast<int64_t>(min(b0 + bl, tile_end - 1)) * row); }

    // group-mean query -> LDS: sequential adds over the g heads of a group, then * (1/g)
    {
        const int g = q_heads / kv_heads;
        const float inv = 1.0f / static_cast<float>(g);
        const QT* qp = q + static_cast<int64_t>(l) * q_layer_stride +
                       q_row * q_heads * kD;
        for (int e = threadIdx.x * 4; e < row; e += kThreads * 4) {
            const int hh = e / kD, d = e - hh * kD;
            const f32x4 mean = group_mean4_any(qp + static_cast<int64_t>(hh) * g * kD + d, kD, g, inv);
            *reinterpret_cast<f32x4*>(&qbar[e]) = mean;
        }
    }
    __syncthreads();

    f32x4 qr[kSteps];
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        qr[i] = *reinterpret_cast<const f32x4*>(&qbar[h * kD + 16 * i + 4 * m]);
    }

    // two passes per trip: the loads of the next pass are in flight while this one is reduced
    auto finish = [&](const f32x4 (&kv)[kSteps], int base) {
        const float dot = quad_dot<kSteps>(qr, kv);
        float s = 0.0f;
        for (int hh = 0; hh < kv_heads; ++hh) {
            const float dh = __shfl(dot, (bl * kv_heads + hh) * 4, 64);
            s = s + fmaxf(-FLT_MAX, dh);
        }
        const int b = base + bl;
        if (b < tile_end && h == 0 && m == 0) { sout[b] = s * scale; }   // (a scale of 1 changes no bit)
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
__global__ __launch_bounds__(kThreads) void score_kernel_bf16(
    const QT* __restrict__ q, int64_t q_layer_stride, const int32_t* __restrict__ q_rows, int q_heads,
    const uint16_t* __restrict__ repre, int64_t repre_layer_stride, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, int n_req, int kv_heads, float* __restrict__ scores,
    int64_t scores_layer_stride, int tile_blocks, float scale)
{
    constexpr int kSteps = kD / 16;
    __shared__ __attribute__((aligned(16))) float qbar[kMaxRow];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l = blockIdx.y;
    int r, tile;
    if (!find_tile(seg_len, n_req, tile_blocks, blockIdx.x, lane, r, tile)) { return; }
    // a row index that came from device memory is followed only inside the layer's query block
    const int64_t q_row = q_rows ? static_cast<int64_t>(q_rows[r]) : r;
    if (q_rows && (q_row < 0 || (q_row + 1) * q_heads * kD > q_layer_stride)) { return; }   // (the whole workgroup)
    const int n = seg_len[r];
    const int tile0 = tile * tile_blocks;
    const int tile_end = min(tile0 + tile_blocks, n);
    const int row = kv_heads * kD;

    const int p = lane & 1;                 // which 8 of the 16 lanes of the dot product
    const int v = lane >> 1;                // vector of this pass: 0..31
    const int blocks_per_pass = 32 / kv_heads;
    const int bl = v / kv_heads;
    const int h = v - bl * kv_heads;
    const int stride = kWaves * blocks_per_pass;
    const int seg0 = seg_off[r];

    const uint16_t* rbase = repre + static_cast<int64_t>(l) * repre_layer_stride +
                            static_cast<int64_t>(seg0) * row + h * kD + 8 * p;
    float* sout = scores + static_cast<int64_t>(l) * scores_layer_stride + seg0;

    // Loads and the store below are unconditional (rows and the output index are clamped to the tile's last
    // block, whose score is then written more than once): an operation skipped on some path would make the
    // compiler wait for everything outstanding, the prefetch included.  The empty asm keeps the compiler from
    // sinking a prefetch down to its use.
    int b0 = tile0 + wave * blocks_per_pass;
    u32x4 kv_a[kSteps], kv_b[kSteps];
    load_pass_bf16<kSteps>(kv_a, rbase + static_cast<int64_t>(min(b0 + bl, tile_end - 1)) * row);
    asm volatile("" ::: "memory");

    {
        const int g = q_heads / kv_heads;
        const float inv = 1.0f / static_cast<float>(g);
        const QT* qp = q + static_cast<int64_t>(l) * q_layer_stride +
                       q_row * q_heads * kD;
        for (int e = threadIdx.x * 4; e < row; e += kThreads * 4) {
            const int hh = e / kD, d = e - hh * kD;
            const f32x4 mean = group_mean4_any(qp + static_cast<int64_t>(hh) * g * kD + d, kD, g, inv);
            *reinterpret_cast<f32x4*>(&qbar[e]) = mean;
        }
    }
    __syncthreads();

    f32x4 qlo[kSteps], qhi[kSteps];
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        qlo[i] = *reinterpret_cast<const f32x4*>(&qbar[h * kD + 16 * i + 8 * p]);
        qhi[i] = *reinterpret_cast<const f32x4*>(&qbar[h * kD + 16 * i + 8 * p + 4]);
    }

    auto finish = [&](const u32x4 (&kv)[kSteps], int base) {
        const float dot = pair_dot<kSteps>(qlo, qhi, kv);
        float s = 0.0f;
        for (int hh = 0; hh < kv_heads; ++hh) {
            const float dh = __shfl(dot, (bl * kv_heads + hh) * 2, 64);
            s = s + fmaxf(-FLT_MAX, dh);
        }
        sout[min(base + bl, tile_end - 1)] = s * scale;   // the lanes of a block all hold its score; a scale of 1 changes no bit
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

template <int kD, typename QT>
void launch_bf16(const void* q, int64_t q_layer_stride, const int32_t* q_rows, int q_heads, const void* repre,
                 int64_t repre_layer_stride, const int32_t* seg_off, const int32_t* seg_len, int n_req,
                 int64_t tile_bound, int n_layers, int kv_heads, float* scores, int64_t scores_layer_stride,
                 int tile_blocks, float scale, hipStream_t stream)
{
    hipLaunchKernelGGL((score_kernel_bf16<kD, QT>), dim3(static_cast<unsigned>(tile_bound), n_layers), dim3(kThreads), 0,
                       stream, static_cast<const QT*>(q), q_layer_stride, q_rows, q_heads,
                       static_cast<const uint16_t*>(repre), repre_layer_stride, seg_off, seg_len, n_req, kv_heads,
                       scores, scores_layer_stride, tile_blocks, scale);
}

template <int kD, typename QT>
void launch(const void* q, int64_t q_layer_stride, const int32_t* q_rows, int q_heads, const void* repre,
            int64_t repre_layer_stride, const int32_t* seg_off, const int32_t* seg_len, int n_req,
            int64_t tile_bound, int n_layers, int kv_heads, float* scores, int64_t scores_layer_stride,
            int tile_blocks, float scale, hipStream_t stream)
{
    hipLaunchKernelGGL((score_kernel<kD, QT>), dim3(static_cast<unsigned>(tile_bound), n_layers), dim3(kThreads), 0,
                       stream, static_cast<const QT*>(q), q_layer_stride, q_rows, q_heads,
                       static_cast<const float*>(repre), repre_layer_stride,
                       seg_off, seg_len, n_req, kv_heads, scores, scores_layer_stride, tile_blocks, scale);
}

}  // namespace

extern "C" int ucm_score_blocks(const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows,
                                int q_heads, const void* repre, int repre_dtype, int64_t repre_layer_stride,
                                const int32_t* seg_off, const int32_t* seg_len, int n_req, int max_seg_len,
                                int64_t total_blocks, int n_layers, int kv_heads, int head_dim, float* scores,
                                int64_t scores_layer_stride, float scale, int tile_blocks_arg, ucm_stream_t stream)
{
    UCM_REQUIRE(std::isfinite(scale), "ucm_score_blocks: scale is not finite");
    UCM_REQUIRE(tile_blocks_arg >= 0 && tile_blocks_arg <= 4096, "ucm_score_blocks: tile_blocks=%d", tile_blocks_arg);
    UCM_REQUIRE(n_req == 0 || max_seg_len == 0 || (q && repre && seg_off && seg_len && scores),
                "ucm_score_blocks: null pointer");
    UCM_REQUIRE(q_dtype == UCM_DTYPE_F32 || q_dtype == UCM_DTYPE_BF16, "ucm_score_blocks: q_dtype=%d", q_dtype);
    UCM_REQUIRE(repre_dtype == UCM_DTYPE_F32 || repre_dtype == UCM_DTYPE_BF16, "ucm_score_blocks: repre_dtype=%d", repre_dtype);
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535,
                "ucm_score_blocks: n_req=%d n_layers=%d", n_req, n_layers);
    UCM_REQUIRE(max_seg_len >= 0 && total_blocks >= 0, "ucm_score_blocks: max_seg_len=%d total_blocks=%lld",
                max_seg_len, static_cast<long long>(total_blocks));
    UCM_REQUIRE(kv_heads > 0 && q_heads >= kv_heads && q_heads % kv_heads == 0,
                "ucm_score_blocks: q_heads=%d kv_heads=%d", q_heads, kv_heads);
    UCM_SUPPORTED(head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128 || head_dim == 192 || head_dim == 256,
                  "ucm_score_blocks: head_dim=%d (32, 64, 96, 128, 192 or 256)", head_dim);
    UCM_SUPPORTED(kv_heads * head_dim <= kMaxRow, "ucm_score_blocks: kv_heads*head_dim=%d (at most %d)", kv_heads * head_dim, kMaxRow);
    UCM_SUPPORTED(kv_heads <= 16 && 16 % kv_heads == 0, "ucm_score_blocks: kv_heads=%d (1, 2, 4, 8 or 16)", kv_heads);
    UCM_REQUIRE(ucm::aligned16(repre) && repre_layer_stride % (repre_dtype == UCM_DTYPE_BF16 ? 8 : 4) == 0,
                "ucm_score_blocks: repre not 16-byte aligned");
    UCM_SUPPORTED(repre_dtype == UCM_DTYPE_F32 || 32 % kv_heads == 0, "ucm_score_blocks: kv_heads=%d", kv_heads);
    UCM_REQUIRE(ucm::aligned16(q) && q_layer_stride % 8 == 0, "ucm_score_blocks: q not 16-byte aligned");
    UCM_REQUIRE(!q_rows || q_layer_stride >= static_cast<int64_t>(q_heads) * head_dim,
                "ucm_score_blocks: with q_rows, q_layer_stride=%lld bounds the rows and must hold at least one",
                static_cast<long long>(q_layer_stride));
    if (n_req == 0 || max_seg_len == 0) { return UCM_OK; }
    hipStream_t s = ucm::as_stream(stream);
    // upper bound of sum(ceil(seg_len / tile)): exact to within n_req when the host knows the total
    const int row_bytes = kv_heads * head_dim * (repre_dtype == UCM_DTYPE_BF16 ? 2 : 4);
    const int tile_blocks = tile_blocks_arg > 0 ? tile_blocks_arg : std::max(8, (128 * 1024) / row_bytes);
    const int64_t per_req = (static_cast<int64_t>(max_seg_len) + tile_blocks - 1) / tile_blocks;
    int64_t tile_bound = per_req * n_req;
    if (total_blocks > 0) { tile_bound = std::min(tile_bound, (total_blocks + tile_blocks - 1) / tile_blocks + n_req); }
    UCM_REQUIRE(tile_bound <= 0x7fffffffll, "ucm_score_blocks: too many tiles for one launch");
#define UCM_SCORE_ARGS q, q_layer_stride, q_rows, q_heads, repre, repre_layer_stride, seg_off, seg_len, n_req, \
                       tile_bound, n_layers, kv_heads, scores, scores_layer_stride, tile_blocks, scale, s
    const bool qf = q_dtype == UCM_DTYPE_F32;
#define UCM_SCORE_DIM(D)                                                                                        \
    do {                                                                                                        \
        if (repre_dtype == UCM_DTYPE_F32) {                                                                     \
            if (qf) { launch<D, float>(UCM_SCORE_ARGS); } else { launch<D, uint16_t>(UCM_SCORE_ARGS); }         \
        } else {                                                                                                \
            if (qf) { launch_bf16<D, float>(UCM_SCORE_ARGS); } else { launch_bf16<D, uint16_t>(UCM_SCORE_ARGS); } \
        }                                                                                                       \
    } while (0)
    switch (head_dim) {
    case 32: UCM_SCORE_DIM(32); break;
    case 64: UCM_SCORE_DIM(64); break;
    case 96: UCM_SCORE_DIM(96); break;
    case 128: UCM_SCORE_DIM(128); break;
    case 192: UCM_SCORE_DIM(192); break;
    default: UCM_SCORE_DIM(256); break;
    }
#undef UCM_SCORE_DIM
#undef UCM_SCORE_ARGS
    UCM_LAUNCH_CHECK("ucm_score_blocks");
}
