// ESA retrieval backend on the GPU: scores of an arbitrary slot list against a
// flat query, then the best k by score in descending order with their scores.
//
// The reference scores each slot with a strictly sequential
//     score = score + q[d] * data[slot][d]        (separate multiply and add)
// so one thread owns one slot and walks its row in order; what is parallel is
// the slots.  Rows are 4 KiB apart, so they are staged through LDS: the four
// waves of a workgroup fetch a 64-row x 128-column tile with coalesced 16-byte
// loads (the next tile's loads are already in flight while the current one is
// consumed), and one wave then reads its row from LDS, conflict-free thanks to
// an odd row stride.  Latency-bound by design (a chain of `dim` dependent adds).
//
// Selection is a bitonic sort of 64-bit keys (order-preserving score bits, then
// position ascending) in LDS, one workgroup per request.
#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSlots = 64;          // slots (rows) per workgroup
constexpr int kCols = 128;          // columns per tile
constexpr int kStride = kCols + 1;  // odd stride: lane r reading column d hits bank (r + d) % 64
constexpr int kScoreThreads = 256;
constexpr int kRowsPerLoad = kScoreThreads / (kCols / 4);  // 8 rows per 16-byte load instruction
constexpr int kLoads = kSlots / kRowsPerLoad;              // 8 loads per thread per tile

// grid: x = group of 64 entries of the index row, y = request
__global__ __launch_bounds__(kScoreThreads) void esa_score_kernel(
    const float* __restrict__ data, unsigned n_items, unsigned dim, const float* __restrict__ q,
    const int32_t* __restrict__ indexes, unsigned m, float* __restrict__ scores)
{
    __shared__ float tile[kSlots * kStride];
    __shared__ int32_t slot_of[kSlots];

    const unsigned b = blockIdx.y, first = blockIdx.x * kSlots;
    const int32_t* idx_row = indexes + static_cast<size_t>(b) * m;
    if (threadIdx.x < kSlots) {
        const unsigned e = first + threadIdx.x;
        const int32_t s = e < m ? idx_row[e] : -1;
        slot_of[threadIdx.x] = (s >= 0 && static_cast<unsigned>(s) < n_items) ? s : -1;
    }
    __syncthreads();

    // this thread's part of a tile: column group c4 (4 floats) of rows r0, r0+8, ...
    const unsigned c4 = threadIdx.x % (kCols / 4), r0 = threadIdx.x / (kCols / 4);
    const float* row_ptr[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int32_t s = slot_of[r0 + i * kRowsPerLoad];
        row_ptr[i] = data + static_cast<size_t>(s < 0 ? 0 : s) * dim + c4 * 4;
    }
    const float* qb = q + static_cast<size_t>(b) * dim;

    f32x4 regs[kLoads];
    auto fetch = [&](unsigned col0) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            if (col0 + c4 * 4 < dim) { regs[i] = *reinterpret_cast<const f32x4*>(row_ptr[i] + col0); }
        }
    };
    fetch(0);
    float score = 0.0f;
    for (unsigned col0 = 0; col0 < dim; col0 += kCols) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            float* t = &tile[(r0 + i * kRowsPerLoad) * kStride + c4 * 4];
            t[0] = regs[i].x; t[1] = regs[i].y; t[2] = regs[i].z; t[3] = regs[i].w;
        }
        __syncthreads();
        if (col0 + kCols < dim) { fetch(col0 + kCols); }
        if (threadIdx.x < kSlots) {
            const unsigned width = min(static_cast<unsigned>(kCols), dim - col0);
            const float* mine = &tile[threadIdx.x * kStride];
            for (unsigned d = 0; d < width; ++d) {
                const float p = qb[col0 + d] * mine[d];
                score = score + p;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x < kSlots && first + threadIdx.x < m) {
        scores[static_cast<size_t>(b) * m + first + threadIdx.x] = score;
    }
}

__device__ __forceinline__ unsigned ordered_key(float f)
{
    f = f + 0.0f;
    const unsigned u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

constexpr int kSortThreads = 1024;

// grid: x = request; dynamic LDS: n_pad 64-bit keys
__global__ __launch_bounds__(kSortThreads) void esa_topk_kernel(
    const float* __restrict__ scores, const int32_t* __restrict__ indexes, unsigned n_items, unsigned m,
    unsigned n_pad, int topk, int32_t* __restrict__ out_idx, float* __restrict__ out_scores,
    int32_t* __restrict__ out_count, unsigned out_stride)
{
    extern __shared__ unsigned long long keys[];
    __shared__ unsigned valid_total;
    const unsigned b = blockIdx.x;
    const float* s_row = scores + static_cast<size_t>(b) * m;
    const int32_t* idx_row = indexes + static_cast<size_t>(b) * m;
    if (threadIdx.x == 0) { valid_total = 0; }
    __syncthreads();
    unsigned mine = 0;
    for (unsigned e = threadIdx.x; e < n_pad; e += kSortThreads) {
        unsigned long long key = 0;  // padding and skipped entries sort last
        if (e < m) {
            const int32_t s = idx_row[e];
            if (s >= 0 && static_cast<unsigned>(s) < n_items) {
                key = (static_cast<unsigned long long>(ordered_key(s_row[e])) << 32) | (0xffffffffu - e);
                ++mine;
            }
        }
        keys[e] = key;
    }
    atomicAdd(&valid_total, mine);
    __syncthreads();

    // bitonic sort, descending
    for (unsigned size = 2; size <= n_pad; size <<= 1) {
        for (unsigned stride = size >> 1; stride > 0; stride >>= 1) {
            for (unsigned t = threadIdx.x; t < n_pad / 2; t += kSortThreads) {
                const unsigned lo = 2 * t - (t & (stride - 1));
                const unsigned hi = lo + stride;
                const bool descending = (lo & size) == 0;
                const unsigned long long a = keys[lo], c = keys[hi];
                if ((a < c) == descending) { keys[lo] = c; keys[hi] = a; }
            }
            __syncthreads();
        }
    }

    const int valid = static_cast<int>(valid_total);
    const int count = max(0, min(valid, topk));
    for (int i = threadIdx.x; i < count; i += kSortThreads) {
        const unsigned e = 0xffffffffu - static_cast<unsigned>(keys[i] & 0xffffffffu);
        out_idx[static_cast<size_t>(b) * out_stride + i] = idx_row[e];
        out_scores[static_cast<size_t>(b) * out_stride + i] = s_row[e];
    }
    if (threadIdx.x == 0) { out_count[b] = count; }
}

}  // namespace

extern "C" int ucm_esa_retrieve(const float* data, int n_items, int dim, const float* q,
                                const int32_t* indexes, int batch, int m, int topk, float* scores_ws,
                                int32_t* out_idx, float* out_scores, int32_t* out_count, int out_stride,
                                ucm_stream_t stream)
{
    UCM_REQUIRE(batch >= 0 && m >= 0, "ucm_esa_retrieve: batch=%d m=%d", batch, m);
    if (batch == 0) { return UCM_OK; }
    UCM_REQUIRE(data && q && out_idx && out_scores && out_count, "ucm_esa_retrieve: null pointer");
    UCM_REQUIRE(m == 0 || (indexes && scores_ws), "ucm_esa_retrieve: null index row or workspace");
    UCM_REQUIRE(n_items > 0 && dim > 0, "ucm_esa_retrieve: n_items=%d dim=%d", n_items, dim);
    UCM_SUPPORTED(dim % 4 == 0, "ucm_esa_retrieve: dim=%d must be a multiple of 4", dim);
    UCM_REQUIRE(ucm::aligned16(data) && ucm::aligned16(q), "ucm_esa_retrieve: data and q must be 16-byte aligned");
    UCM_REQUIRE(batch <= 65535, "ucm_esa_retrieve: batch=%d", batch);
    UCM_REQUIRE(out_stride >= std::min(std::max(topk, 0), m), "ucm_esa_retrieve: out_stride=%d too small", out_stride);
    unsigned n_pad = 2;
    while (n_pad < static_cast<unsigned>(m)) { n_pad <<= 1; }
    UCM_SUPPORTED(n_pad <= 8192, "ucm_esa_retrieve: m=%d (at most 8192 candidates per request)", m);
    hipStream_t s = ucm::as_stream(stream);
    if (m > 0) {
        hipLaunchKernelGGL(esa_score_kernel, dim3((m + kSlots - 1) / kSlots, batch), dim3(kScoreThreads), 0, s,
                           data, static_cast<unsigned>(n_items), static_cast<unsigned>(dim), q, indexes,
                           static_cast<unsigned>(m), scores_ws);
        if (int rc = ucm::check_hip(hipGetLastError(), "ucm_esa_retrieve(score)")) { return rc; }
    }
    hipLaunchKernelGGL(esa_topk_kernel, dim3(batch), dim3(kSortThreads), n_pad * sizeof(unsigned long long), s,
                       scores_ws, indexes, static_cast<unsigned>(n_items), static_cast<unsigned>(m), n_pad, topk,
                       out_idx, out_scores, out_count, static_cast<unsigned>(out_stride));
    UCM_LAUNCH_CHECK("ucm_esa_retrieve(select)");
}
