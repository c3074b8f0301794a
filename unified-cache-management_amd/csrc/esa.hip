// ESA retrieval backend on the GPU: scores of an arbitrary slot list against a
// flat query, then the best k by score in descending order with their scores.
//
// The reference scores each slot with a strictly sequential
//     score = score + q[d] * data[slot][d]        (separate multiply and add)
// The products do not depend on the order, the additions do: every thread of a
// workgroup multiplies the 16-byte pieces it fetches (coalesced, rows are 4 KiB
// apart) by the query and parks the products in LDS, column-major with an odd
// column stride, and one wave then adds its slot's products in order - per
// dimension one LDS read at a constant offset and one dependent add, nothing
// else.  Two product tiles alternate, so the other waves fill the next tile
// while the chain of the current one runs, and the loads of the tile after that
// are in flight.  Latency-bound by design (a chain of `dim` dependent adds).
//
// Selection ranks 64-bit keys (order-preserving score bits, then position
// ascending) by counting the keys above each, spread over workgroups.
#include "common.h"

#include <algorithm>
#include <mutex>

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSlots = 64;          // slots (rows) per workgroup
constexpr int kCols = 128;          // columns per tile
constexpr int kColStride = kSlots + 1;  // odd: lane r reading column d hits bank (r + d) % 64
constexpr int kScoreThreads = 256;
constexpr int kRowsPerLoad = kScoreThreads / (kCols / 4);  // 8 rows per 16-byte load instruction
constexpr int kLoads = kSlots / kRowsPerLoad;              // 8 loads per thread per tile
constexpr int kDepth = 2;                                  // tiles in flight per thread (an even number: two LDS buffers)

// Row of the index matrix (and of every per-request output) that request b uses: b itself, or rows[b] when the
// caller keeps a persistent table of requests and a call covers some of them.  A row outside the table makes
// the whole request a no-op.
__device__ __forceinline__ bool request_row(const int32_t* __restrict__ rows, unsigned n_rows, unsigned b, unsigned& row)
{
    if (!rows) { row = b; return true; }
    const int32_t r = rows[b];
    row = static_cast<unsigned>(r);
    return r >= 0 && row < n_rows;
}

// grid: x = group of 64 entries of the index row, y = request
__global__ __launch_bounds__(kScoreThreads) void esa_score_kernel(
    const float* __restrict__ data, unsigned n_items, unsigned dim, const float* __restrict__ q,
    const int32_t* __restrict__ indexes, unsigned m, float* __restrict__ scores,
    const int32_t* __restrict__ rows, unsigned n_rows, unsigned idx_stride)
{
    __shared__ float tile[2][kCols * kColStride];       // products, [column][slot]
    __shared__ int32_t slot_of[kSlots];

    const unsigned b = blockIdx.y, first = blockIdx.x * kSlots;
    unsigned row;
    if (!request_row(rows, n_rows, b, row)) { return; }   // (uniform)
    const int32_t* idx_row = indexes + static_cast<size_t>(row) * idx_stride;
    int32_t my_slot = -1;
    if (threadIdx.x < kSlots) {
        const unsigned e = first + threadIdx.x;
        const int32_t s = e < m ? idx_row[e] : -1;
        my_slot = (s >= 0 && static_cast<unsigned>(s) < n_items) ? s : -1;
        slot_of[threadIdx.x] = my_slot;
    }
    // a group of padding only (short requests in a wide table) has nothing to score: the selection ignores the
    // scores of entries without a slot
    if (!__syncthreads_or(my_slot >= 0)) { return; }

    // this thread's part of a tile: column group c4 (4 floats) of rows r0, r0+8, ...
    const unsigned c4 = threadIdx.x % (kCols / 4), r0 = threadIdx.x / (kCols / 4);
    const float* row_ptr[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int32_t s = slot_of[r0 + i * kRowsPerLoad];
        row_ptr[i] = data + static_cast<size_t>(s < 0 ? 0 : s) * dim + c4 * 4;
    }
    const float* qb = q + static_cast<size_t>(b) * dim + c4 * 4;

    // kDepth tiles of loads are in flight per thread: a tile's chain (128 dependent adds) is several times
    // shorter than a trip to memory, so the chain of tile t runs while tiles t+1 .. t+kDepth-1 are on their way
    f32x4 regs[kDepth][kLoads], qv[kDepth];
    auto fetch = [&](int stage, unsigned col0) {
        if (col0 + c4 * 4 < dim) {
            qv[stage] = *reinterpret_cast<const f32x4*>(qb + col0);
#pragma unroll
            for (int i = 0; i < kLoads; ++i) { regs[stage][i] = *reinterpret_cast<const f32x4*>(row_ptr[i] + col0); }
        }
    };
#pragma unroll
    for (int u = 0; u < kDepth; ++u) {
        if (u * kCols < dim) { fetch(u, u * kCols); }
    }
    float score = 0.0f;
    for (unsigned base = 0; base < dim; base += kDepth * kCols) {
#pragma unroll
        for (int u = 0; u < kDepth; ++u) {
            const unsigned col0 = base + u * kCols;
            if (col0 >= dim) { break; }                  // (uniform)
            // (tiles alternate between two buffers; a buffer is rewritten two tiles later, after the barrier
            // of the tile in between, which the chain wave only reaches when its chain is done)
            float* tb = tile[u & 1];
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                float* t = &tb[(c4 * 4) * kColStride + r0 + i * kRowsPerLoad];
                t[0] = qv[u].x * regs[u][i].x;
                t[kColStride] = qv[u].y * regs[u][i].y;
                t[2 * kColStride] = qv[u].z * regs[u][i].z;
                t[3 * kColStride] = qv[u].w * regs[u][i].w;
            }
            __syncthreads();
            if (col0 + kDepth * kCols < dim) { fetch(u, col0 + kDepth * kCols); }
            if (threadIdx.x < kSlots) {
                const float* mine = &tb[threadIdx.x];
                if (col0 + kCols <= dim) {
#pragma unroll 32
                    for (int d = 0; d < kCols; ++d) { score = score + mine[d * kColStride]; }
                } else {
                    for (unsigned d = 0; d < dim - col0; ++d) { score = score + mine[d * kColStride]; }
                }
            }
        }
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

constexpr int kRankThreads = 256;

// Selection by counting: keys are distinct (the position is part of the key), so a candidate's place in
// the descending order is the number of keys above its own.  Every workgroup builds all keys of its request
// in LDS; kLanes lanes share a candidate, each counting over every kLanes-th key (lanes of a wave read at
// most kLanes different addresses at a time, the rest are broadcasts), and the best `topk` candidates write
// themselves to their places.  No sorting network, no barrier after the keys are built; long candidate lists
// spread over many workgroups.
// grid: x = group of 256/kLanes candidates, y = request; dynamic LDS: n_pad 64-bit keys
template <int kLanes>
__global__ __launch_bounds__(kRankThreads) void esa_rank_kernel(
    const float* __restrict__ scores, const int32_t* __restrict__ indexes, unsigned n_items, unsigned m,
    unsigned n_pad, int topk, int32_t* __restrict__ out_idx, float* __restrict__ out_scores,
    int32_t* __restrict__ out_count, unsigned out_stride, const int32_t* __restrict__ rows, unsigned n_rows,
    const int32_t* __restrict__ topk_rows, int32_t* __restrict__ out_pos, unsigned idx_stride)
{
    extern __shared__ __attribute__((aligned(16))) unsigned long long keys[];
    __shared__ unsigned valid_total;
    const unsigned b = blockIdx.y;
    unsigned row;
    if (!request_row(rows, n_rows, b, row)) { return; }   // (uniform)
    if (topk_rows) { topk = min(topk, topk_rows[row]); }  // the request's own k, never beyond a row of the outputs
    const float* s_row = scores + static_cast<size_t>(b) * m;
    const int32_t* idx_row = indexes + static_cast<size_t>(row) * idx_stride;
    if (threadIdx.x == 0) { valid_total = 0; }
    __syncthreads();
    unsigned mine = 0;
    for (unsigned e0 = threadIdx.x; e0 < n_pad; e0 += 8 * kRankThreads) {
        int32_t slot[8];
        float sc[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {                    // both loads of all eight entries at once
            const unsigned e = e0 + u * kRankThreads;
            slot[u] = e < m ? idx_row[e] : -1;
            sc[u] = e < m ? s_row[e] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const unsigned e = e0 + u * kRankThreads;
            unsigned long long key = 0;  // padding and skipped entries: below every candidate
            if (slot[u] >= 0 && static_cast<unsigned>(slot[u]) < n_items) {
                key = (static_cast<unsigned long long>(ordered_key(sc[u])) << 32) | (0xffffffffu - e);
                ++mine;
            }
            if (e < n_pad) { keys[e] = key; }
        }
    }
    if (blockIdx.x == 0) { atomicAdd(&valid_total, mine); }
    __syncthreads();
    if (blockIdx.x == 0 && threadIdx.x == 0) { out_count[row] = max(0, min(static_cast<int>(valid_total), topk)); }

    const unsigned cand = blockIdx.x * (kRankThreads / kLanes) + threadIdx.x / kLanes, sub = threadIdx.x % kLanes;
    const unsigned long long my = cand < m ? keys[cand] : 0ull;
    // two keys per 16-byte read, eight reads in flight; n_pad is a multiple of 16 * kLanes
    typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
    const u64x2* pairs = reinterpret_cast<const u64x2*>(keys);
    unsigned above = 0;
    for (unsigned j = sub; j < n_pad / 2; j += 8 * kLanes) {
        u64x2 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) { v[u] = pairs[j + u * kLanes]; }
#pragma unroll
        for (int u = 0; u < 8; ++u) { above += (v[u].x > my ? 1u : 0u) + (v[u].y > my ? 1u : 0u); }
    }
#pragma unroll
    for (int d = 1; d < kLanes; d <<= 1) { above += __shfl_xor(above, d, 64); }
    if (sub == 0 && my != 0ull && static_cast<int>(above) < topk) {      // (a valid key is never zero)
        out_idx[static_cast<size_t>(row) * out_stride + above] = idx_row[cand];
        out_scores[static_cast<size_t>(row) * out_stride + above] = s_row[cand];
        if (out_pos) { out_pos[static_cast<size_t>(row) * out_stride + above] = static_cast<int32_t>(cand); }
    }
}

}  // namespace

// Scratch of ucm_esa_retrieve_static: the candidate scores of one call (what the scores_ws argument of
// ucm_esa_retrieve brings in).  Every GPU holds its own copy of the array at its own address, until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kStaticScoreFloats = size_t{1} << 19;   // 2 MiB: e.g. 64 requests x 8192 candidates
static __device__ __align__(256) float scratch[kStaticScoreFloats];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch` on each GPU, looked up once per GPU

// Device address of the current GPU's copy of `scratch` (first call on a GPU: one symbol lookup, no allocation).
int static_scratch(float** out)
{
    int dev = -1;
    if (int rc = ucm::check_hip(hipGetDevice(&dev), "ucm_esa_retrieve_static(hipGetDevice)")) { return rc; }
    if (dev < 0 || dev >= kMaxDevices) { return ucm::fail(UCM_ENOTSUP, "ucm_esa_retrieve_static: device %d (at most %d)", dev, kMaxDevices); }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        if (int rc = ucm::check_hip(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)),
                                    "ucm_esa_retrieve_static(hipGetSymbolAddress)")) {
            return rc;
        }
        if (!ptr) { return ucm::fail(UCM_EHIP, "ucm_esa_retrieve_static: no device address for the scratch array"); }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return UCM_OK;
}

int esa_retrieve_impl(const char* name, const float* data, int n_items, int dim, const float* q, const int32_t* indexes,
                      int batch, int m, int topk, float* scores_ws, int32_t* out_idx, float* out_scores,
                      int32_t* out_count, int out_stride, ucm_stream_t stream, const int32_t* rows = nullptr,
                      int n_rows = 0, const int32_t* topk_rows = nullptr, int32_t* out_pos = nullptr, int idx_stride = -1)
{
    const unsigned stride = static_cast<unsigned>(idx_stride < 0 ? m : idx_stride);   // row pitch of the index matrix
    const unsigned n_pad = (static_cast<unsigned>(m) + 127u) & ~127u;    // whole rounds of the counting loop
    hipStream_t s = ucm::as_stream(stream);
    if (m > 0) {
        hipLaunchKernelGGL(esa_score_kernel, dim3((m + kSlots - 1) / kSlots, batch), dim3(kScoreThreads), 0, s,
                           data, static_cast<unsigned>(n_items), static_cast<unsigned>(dim), q, indexes,
                           static_cast<unsigned>(m), scores_ws, rows, static_cast<unsigned>(n_rows), stride);
        if (int rc = ucm::check_hip(hipGetLastError(), name)) { return rc; }
    }
    if (m <= 1024) {
        hipLaunchKernelGGL(esa_rank_kernel<1>, dim3((m + kRankThreads - 1) / kRankThreads + (m == 0), batch), dim3(kRankThreads),
                           n_pad * sizeof(unsigned long long), s, scores_ws, indexes, static_cast<unsigned>(n_items),
                           static_cast<unsigned>(m), n_pad, topk, out_idx, out_scores, out_count, static_cast<unsigned>(out_stride),
                           rows, static_cast<unsigned>(n_rows), topk_rows, out_pos, stride);
    } else {
        constexpr int kPer = kRankThreads / 8;
        hipLaunchKernelGGL(esa_rank_kernel<8>, dim3((m + kPer - 1) / kPer, batch), dim3(kRankThreads),
                           n_pad * sizeof(unsigned long long), s, scores_ws, indexes, static_cast<unsigned>(n_items),
                           static_cast<unsigned>(m), n_pad, topk, out_idx, out_scores, out_count, static_cast<unsigned>(out_stride),
                           rows, static_cast<unsigned>(n_rows), topk_rows, out_pos, stride);
    }
    return ucm::check_hip(hipGetLastError(), name);
}

}  // namespace

#define UCM_ESA_CHECK_ARGS(name, ws_ok)                                                                              \
    UCM_REQUIRE(batch >= 0 && m >= 0, name ": batch=%d m=%d", batch, m);                                             \
    if (batch == 0) { return UCM_OK; }                                                                               \
    UCM_REQUIRE(data && q && out_idx && out_scores && out_count, name ": null pointer");                             \
    UCM_REQUIRE(m == 0 || (indexes && (ws_ok)), name ": null index row or workspace");                               \
    UCM_REQUIRE(n_items > 0 && dim > 0, name ": n_items=%d dim=%d", n_items, dim);                                   \
    UCM_SUPPORTED(dim % 4 == 0, name ": dim=%d must be a multiple of 4", dim);                                       \
    UCM_REQUIRE(ucm::aligned16(data) && ucm::aligned16(q), name ": data and q must be 16-byte aligned");             \
    UCM_REQUIRE(batch <= 65535, name ": batch=%d", batch);                                                           \
    UCM_REQUIRE(out_stride >= std::min(std::max(topk, 0), m), name ": out_stride=%d too small", out_stride);         \
    UCM_SUPPORTED(m <= 8192, name ": m=%d (at most 8192 candidates per request)", m)

extern "C" int ucm_esa_retrieve(const float* data, int n_items, int dim, const float* q,
                                const int32_t* indexes, int batch, int m, int topk, float* scores_ws,
                                int32_t* out_idx, float* out_scores, int32_t* out_count, int out_stride,
                                ucm_stream_t stream)
{
    UCM_ESA_CHECK_ARGS("ucm_esa_retrieve", scores_ws != nullptr);
    return esa_retrieve_impl("ucm_esa_retrieve", data, n_items, dim, q, indexes, batch, m, topk, scores_ws, out_idx,
                             out_scores, out_count, out_stride, stream);
}

extern "C" int ucm_esa_retrieve_static(const float* data, int n_items, int dim, const float* q,
                                       const int32_t* indexes, int batch, int m, int topk, int32_t* out_idx,
                                       float* out_scores, int32_t* out_count, int out_stride, ucm_stream_t stream)
{
    UCM_ESA_CHECK_ARGS("ucm_esa_retrieve_static", true);
    UCM_SUPPORTED(static_cast<size_t>(batch) * static_cast<size_t>(m) <= kStaticScoreFloats,
                  "ucm_esa_retrieve_static: batch*m = %zu candidate scores exceed the built-in scratch of %zu "
                  "(use ucm_esa_retrieve with a workspace of its own)",
                  static_cast<size_t>(batch) * static_cast<size_t>(m), kStaticScoreFloats);
    float* ws = nullptr;
    if (int rc = static_scratch(&ws)) { return rc; }
    return esa_retrieve_impl("ucm_esa_retrieve_static", data, n_items, dim, q, indexes, batch, m, topk, ws, out_idx,
                             out_scores, out_count, out_stride, stream);
}

extern "C" int ucm_esa_retrieve_rows(const float* data, int n_items, int dim, const float* q,
                                     const int32_t* slot_table, int table_rows, int table_stride, int m,
                                     const int32_t* rows, int batch, const int32_t* topk_rows, int max_topk,
                                     float* scores_ws, int32_t* out_idx, int32_t* out_pos, float* out_scores,
                                     int32_t* out_count, int out_stride, ucm_stream_t stream)
{
    const int topk = max_topk;
    const int32_t* indexes = slot_table;
    UCM_ESA_CHECK_ARGS("ucm_esa_retrieve_rows", scores_ws != nullptr);
    UCM_REQUIRE(rows && topk_rows && table_rows > 0 && table_stride >= m,
                "ucm_esa_retrieve_rows: rows, topk_rows, table_rows and table_stride >= m are required");
    return esa_retrieve_impl("ucm_esa_retrieve_rows", data, n_items, dim, q, slot_table, batch, m, max_topk, scores_ws,
                             out_idx, out_scores, out_count, out_stride, stream, rows, table_rows, topk_rows, out_pos,
                             table_stride);
}
