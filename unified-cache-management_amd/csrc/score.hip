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
#include <cfloat>

#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxRow = 16 * 128;  // kv_heads <= 16, head_dim <= 128

template <int kCtrl>
__device__ __forceinline__ float quad_perm(float x)
{
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), kCtrl, 0xf, 0xf, true));
}
constexpr int kQuadXor2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kQuadXor1 = 0xB1;  // quad_perm:[1,0,3,2]

__device__ __forceinline__ float load_q(const float* p) { return *p; }
__device__ __forceinline__ float load_q(const uint16_t* p) { return __uint_as_float(static_cast<unsigned>(*p) << 16); }

// grid: x = tile of `tile_blocks` blocks, y = request, z = layer
template <int kD, typename QT>
__global__ __launch_bounds__(kThreads) void score_kernel(
    const QT* __restrict__ q, int64_t q_layer_stride, const int32_t* __restrict__ q_rows, int q_heads,
    const float* __restrict__ repre, int64_t repre_layer_stride, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, int kv_heads, float* __restrict__ scores,
    int64_t scores_layer_stride, int tile_blocks)
{
    constexpr int kSteps = kD / 16;
    __shared__ float qbar[kMaxRow];

    const int r = blockIdx.y, l = blockIdx.z;
    const int n = seg_len[r];
    const int tile0 = blockIdx.x * tile_blocks;
    if (tile0 >= n) { return; }
    const int tile_end = min(tile0 + tile_blocks, n);
    const int row = kv_heads * kD;

    // group-mean query: sequential adds over the g heads of a group, then * (1/g)
    {
        const int g = q_heads / kv_heads;
        const float inv = 1.0f / static_cast<float>(g);
        const QT* qp = q + static_cast<int64_t>(l) * q_layer_stride +
                       static_cast<int64_t>(q_rows ? q_rows[r] : r) * q_heads * kD;
        for (int e = threadIdx.x; e < row; e += kThreads) {
            const int h = e / kD, d = e - h * kD;
            const QT* src = qp + static_cast<int64_t>(h) * g * kD + d;
            float acc = load_q(src);
            for (int j = 1; j < g; ++j) { acc = acc + load_q(src + j * kD); }
            qbar[e] = g == 1 ? acc : acc * inv;
        }
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 3;                 // which 4 of the 16 lanes of the dot product
    const int v = lane >> 2;                // vector of this pass: 0..15
    const int blocks_per_pass = 16 / kv_heads;
    const int bl = v / kv_heads;            // block within the pass
    const int h = v - bl * kv_heads;        // kv head, fixed for the whole kernel

    f32x4 qr[kSteps];
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
        qr[i] = *reinterpret_cast<const f32x4*>(&qbar[h * kD + 16 * i + 4 * m]);
    }

    const float* rbase = repre + static_cast<int64_t>(l) * repre_layer_stride +
                         static_cast<int64_t>(seg_off[r]) * row + h * kD + 4 * m;
    float* sout = scores + static_cast<int64_t>(l) * scores_layer_stride + seg_off[r];

    for (int b0 = tile0 + wave * blocks_per_pass; b0 < tile_end; b0 += kWaves * blocks_per_pass) {
        const int b = b0 + bl;
        const bool valid = b < tile_end;
        const float* p = rbase + static_cast<int64_t>(valid ? b : b0) * row;
        f32x4 kv[kSteps];
#pragma unroll
        for (int i = 0; i < kSteps; ++i) {
            kv[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + 16 * i));
        }
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
        const float dot = (a0 + a2) + (a1 + a3);

        float s = 0.0f;
        for (int hh = 0; hh < kv_heads; ++hh) {
            const float dh = __shfl(dot, (bl * kv_heads + hh) * 4, 64);
            s = s + fmaxf(-FLT_MAX, dh);
        }
        if (valid && h == 0 && m == 0) { sout[b] = s; }
    }
}

template <int kD, typename QT>
void launch(const void* q, int64_t q_layer_stride, const int32_t* q_rows, int q_heads, const float* repre,
            int64_t repre_layer_stride, const int32_t* seg_off, const int32_t* seg_len, int n_req,
            int max_seg_len, int n_layers, int kv_heads, float* scores, int64_t scores_layer_stride,
            int tile_blocks, hipStream_t stream)
{
    const unsigned tiles = static_cast<unsigned>((max_seg_len + tile_blocks - 1) / tile_blocks);
    hipLaunchKernelGGL((score_kernel<kD, QT>), dim3(tiles, n_req, n_layers), dim3(kThreads), 0, stream,
                       static_cast<const QT*>(q), q_layer_stride, q_rows, q_heads, repre, repre_layer_stride,
                       seg_off, seg_len, kv_heads, scores, scores_layer_stride, tile_blocks);
}

int g_tile_blocks = 32;

}  // namespace

// Tuning knob for benchmarks: blocks scored per workgroup (default 32).
extern "C" int ucm_set_score_tile(int tile_blocks)
{
    UCM_REQUIRE(tile_blocks >= 1 && tile_blocks <= 4096, "ucm_set_score_tile: %d", tile_blocks);
    g_tile_blocks = tile_blocks;
    return UCM_OK;
}

extern "C" int ucm_score_blocks(const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows,
                                int q_heads, const float* repre, int64_t repre_layer_stride,
                                const int32_t* seg_off, const int32_t* seg_len, int n_req, int max_seg_len,
                                int n_layers, int kv_heads, int head_dim, float* scores,
                                int64_t scores_layer_stride, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req == 0 || max_seg_len == 0 || (q && repre && seg_off && seg_len && scores),
                "ucm_score_blocks: null pointer");
    UCM_REQUIRE(q_dtype == UCM_DTYPE_F32 || q_dtype == UCM_DTYPE_BF16, "ucm_score_blocks: q_dtype=%d", q_dtype);
    UCM_REQUIRE(n_req >= 0 && n_req <= 65535 && n_layers > 0 && n_layers <= 65535,
                "ucm_score_blocks: n_req=%d n_layers=%d", n_req, n_layers);
    UCM_REQUIRE(max_seg_len >= 0, "ucm_score_blocks: max_seg_len=%d", max_seg_len);
    UCM_REQUIRE(kv_heads > 0 && q_heads >= kv_heads && q_heads % kv_heads == 0,
                "ucm_score_blocks: q_heads=%d kv_heads=%d", q_heads, kv_heads);
    UCM_SUPPORTED(head_dim == 64 || head_dim == 128, "ucm_score_blocks: head_dim=%d (64 or 128)", head_dim);
    UCM_SUPPORTED(kv_heads <= 16 && 16 % kv_heads == 0, "ucm_score_blocks: kv_heads=%d (1, 2, 4, 8 or 16)", kv_heads);
    UCM_REQUIRE(ucm::aligned16(repre) && repre_layer_stride % 4 == 0, "ucm_score_blocks: repre not 16-byte aligned");
    if (n_req == 0 || max_seg_len == 0) { return UCM_OK; }
    hipStream_t s = ucm::as_stream(stream);
#define UCM_SCORE_ARGS q, q_layer_stride, q_rows, q_heads, repre, repre_layer_stride, seg_off, seg_len, n_req, \
                       max_seg_len, n_layers, kv_heads, scores, scores_layer_stride, g_tile_blocks, s
    if (head_dim == 128) {
        if (q_dtype == UCM_DTYPE_F32) { launch<128, float>(UCM_SCORE_ARGS); } else { launch<128, uint16_t>(UCM_SCORE_ARGS); }
    } else {
        if (q_dtype == UCM_DTYPE_F32) { launch<64, float>(UCM_SCORE_ARGS); } else { launch<64, uint16_t>(UCM_SCORE_ARGS); }
    }
#undef UCM_SCORE_ARGS
    UCM_LAUNCH_CHECK("ucm_score_blocks");
}
