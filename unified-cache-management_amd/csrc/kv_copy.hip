// Paged-KV block moves: pointer-array batch copy, block-id driven dump/load in
// the stored-block layout, and the gather of selected blocks from a device
// block table.  Pure HBM traffic: every byte is read once and written once, so
// the kernels are 16-byte vector copies with non-temporal hints, one
// 1024-thread workgroup per slice (a 256 KiB K or V block = 2 trips of 128 KiB
// in flight), launched with far more workgroups than the 256 CUs.  Of the
// shapes tried on MI355X (8 KiB .. 256 KiB per workgroup, 64 .. 1024 threads,
// 1 .. 16 loads in flight per thread, persistent grids, with and without the
// non-temporal hint) this one was the fastest; all of them sit between 5.2 and
// 6.0 TB/s for a 1:1 read/write mix.
#include "common.h"

namespace {

using ucm::u32x4;

constexpr int kThreads = 1024;
constexpr int kUnroll = 8;
constexpr size_t kStep = static_cast<size_t>(kThreads) * 16 * kUnroll;  // 128 KiB per trip

// kN x 16 KiB of a slice: every load is issued before the first store goes out.  Stores that start as the
// loads trickle in mix reads and writes on the HBM channels and cost about 6 % of the copy rate (1.64 ms ->
// 1.75 ms for the 5.1 GB gather), hence the wait for ALL of the trip's loads.
template <int kN>
__device__ __forceinline__ void copy_trip(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, size_t base)
{
    u32x4 v[kN];
#pragma unroll
    for (int u = 0; u < kN; ++u) {
        v[u] = ucm::gload16_nt(src + base + static_cast<size_t>(u) * kThreads * 16);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int u = 0; u < kN; ++u) {
        ucm::gstore16_nt(dst + base + static_cast<size_t>(u) * kThreads * 16, v[u]);
    }
}

// One workgroup copies one whole slice (a 256 KiB K or V block = 2 trips of 128 KiB).  size is a multiple of
// 16.  What is left after the 128 KiB trips goes in trips of 64, 32 and 16 KiB (the slices of 64-, 32- and
// 16-token blocks), each with all its loads in flight at once, and a last partial one.
__device__ __forceinline__ void copy_slice(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, size_t size)
{
    size_t o = 0;
    const size_t mine = threadIdx.x * 16u;
    for (; o + kStep <= size; o += kStep) { copy_trip<kUnroll>(dst, src, o + mine); }
    if (o + kStep / 2 <= size) { copy_trip<kUnroll / 2>(dst, src, o + mine); o += kStep / 2; }
    if (o + kStep / 4 <= size) { copy_trip<kUnroll / 4>(dst, src, o + mine); o += kStep / 4; }
    if (o + kStep / 8 <= size) { copy_trip<kUnroll / 8>(dst, src, o + mine); o += kStep / 8; }
    if (o + mine < size) { ucm::gstore16_nt(dst + o + mine, ucm::gload16_nt(src + o + mine)); }
}

__global__ __launch_bounds__(kThreads) void copy_batch_kernel(void* const* __restrict__ dst,
                                                              const void* const* __restrict__ src,
                                                              size_t size, size_t piece)
{
    // large copies are cut into pieces so that one pointer pair still fills the chip
    const size_t pieces = (size + piece - 1) / piece;
    const size_t i = blockIdx.x / pieces, c = blockIdx.x % pieces;
    const size_t off = c * piece;
    const size_t len = off + piece <= size ? piece : size - off;
    copy_slice(static_cast<uint8_t*>(dst[i]) + off, static_cast<const uint8_t*>(src[i]) + off, len);
}

// Where a cache block's K and V slices of a layer sit inside a stored block: at layer * layer_pitch + slice_base
// (K) and block_bytes later (V).  One rank's blocks: layer_pitch = 2 * block_bytes, slice_base = 0; rank r of tp
// ranks that share the stored block: layer_pitch = 2 * block_bytes * tp, slice_base = 2 * block_bytes * r.
struct StoredLayout {
    size_t layer_pitch, slice_base;
    __host__ __device__ size_t slice(size_t layer, unsigned kv, size_t block_bytes) const
    {
        return layer * layer_pitch + slice_base + kv * block_bytes;
    }
};

// grid: x = index into block_ids, y = layer, z = K|V
template <bool kToStaging>
__global__ __launch_bounds__(kThreads) void kv_blocks_kernel(void* const* __restrict__ layers,
                                                             size_t kv_stride, size_t block_bytes,
                                                             const int32_t* __restrict__ block_ids,
                                                             unsigned num_blocks,
                                                             uint8_t* __restrict__ staging, StoredLayout lay)
{
    const unsigned i = blockIdx.x, l = blockIdx.y, kv = blockIdx.z, n_layers = gridDim.y;
    const unsigned id = static_cast<unsigned>(block_ids[i]);
    if (id >= num_blocks) { return; }  // ids outside the cache are skipped, never dereferenced
    uint8_t* cache = static_cast<uint8_t*>(layers[l]) + kv * kv_stride +
                     static_cast<size_t>(id) * block_bytes;
    uint8_t* stage = staging + static_cast<size_t>(i) * n_layers * lay.layer_pitch + lay.slice(l, kv, block_bytes);
    if (kToStaging) { copy_slice(stage, cache, block_bytes); }
    else { copy_slice(cache, stage, block_bytes); }
}

// grid: x = position in the request's selection, y = request, z = layer*2 + K|V
__global__ __launch_bounds__(kThreads) void kv_gather_selected_kernel(
    const void* const* __restrict__ layers, size_t kv_stride, size_t block_bytes,
    const int32_t* __restrict__ phys, const int32_t* __restrict__ count, unsigned num_blocks,
    unsigned n_req, unsigned phys_stride, const int64_t* __restrict__ dst_off,
    const int32_t* __restrict__ region_k, uint8_t* __restrict__ staging, uint64_t staging_blocks)
{
    const unsigned j = blockIdx.x, r = blockIdx.y, l = blockIdx.z >> 1, kv = blockIdx.z & 1;
    const size_t lr = static_cast<size_t>(l) * n_req + r;
    if (static_cast<int32_t>(j) >= count[lr]) { return; }
    const unsigned id = static_cast<unsigned>(phys[lr * phys_stride + j]);
    if (id >= num_blocks) { return; }
    const uint8_t* src = static_cast<const uint8_t*>(layers[l]) + kv * kv_stride +
                         static_cast<size_t>(id) * block_bytes;
    const int64_t off = dst_off[r], region = region_k[r];
    if (off < 0 || region < 0) { return; }
    const uint64_t slot = static_cast<uint64_t>(off) + (static_cast<uint64_t>(l) * 2 + kv) * static_cast<uint64_t>(region) + j;
    if (slot >= staging_blocks) { return; }              // never write outside the staging buffer
    copy_slice(staging + slot * block_bytes, src, block_bytes);
}

// Loads planned on the device: slot j of request row `row` receives logical block load_sel[l][row][j] (or
// nothing, -1) from a pool of stored blocks laid out [block][layer][K|V].
// grid: x = slot (stepping by the grid: most slots of most rows have nothing to load, and a workgroup of this
// size that only finds that out costs microseconds), y = request of the call, z = layer*2 + K|V
__global__ __launch_bounds__(kThreads) void kv_load_planned_kernel(
    void* const* __restrict__ layers, size_t kv_stride, size_t block_bytes, unsigned num_blocks,
    const uint8_t* __restrict__ pool, uint64_t pool_blocks, size_t pool_block_bytes, unsigned store_first_layer,
    const int32_t* __restrict__ load_sel, unsigned n_slots, const int32_t* __restrict__ src_table, unsigned src_stride,
    const int32_t* __restrict__ dst_table, unsigned dst_stride, int64_t dst_layer_stride,
    const int32_t* __restrict__ load_count, const int32_t* __restrict__ rows, unsigned table_rows, StoredLayout lay)
{
    const unsigned b = blockIdx.y, l = blockIdx.z >> 1, kv = blockIdx.z & 1;
    unsigned row = b;
    if (rows) {
        const int32_t r = rows[b];
        if (r < 0) { return; }
        row = static_cast<unsigned>(r);
    }
    if (row >= table_rows) { return; }
    unsigned limit = n_slots;
    if (load_count) { limit = min(limit, static_cast<unsigned>(max(load_count[static_cast<size_t>(l) * table_rows + row], 0))); }
    for (unsigned j = blockIdx.x; j < limit; j += gridDim.x) {    // (uniform: every thread of the workgroup takes the same trips)
        const int32_t sel = load_sel[(static_cast<size_t>(l) * table_rows + row) * n_slots + j];
        if (sel < 0 || static_cast<unsigned>(sel) >= src_stride) { continue; }     // slot keeps what it holds
        const int32_t src = src_table[static_cast<size_t>(row) * src_stride + sel];
        if (src < 0 || static_cast<uint64_t>(src) >= pool_blocks) { continue; }   // block not in the pool
        const unsigned dst = static_cast<unsigned>(dst_table[l * dst_layer_stride + static_cast<int64_t>(row) * dst_stride + j]);
        if (dst >= num_blocks) { continue; }
        copy_slice(static_cast<uint8_t*>(layers[l]) + kv * kv_stride + static_cast<size_t>(dst) * block_bytes,
                   pool + static_cast<size_t>(src) * pool_block_bytes + lay.slice(store_first_layer + l, kv, block_bytes),
                   block_bytes);
    }
}

// The same loads when every row says how many of its leading entries are loads (load_count): the work is
// known exactly, so it is dealt out evenly.  Every workgroup builds the running total of the (layer, request)
// pairs' counts in LDS (a few hundred integers), and takes the copies w, w + grid, ... of the 2 * total
// (K and V); which pair a copy belongs to is a binary search in the totals.  grid: x = workgroup.
constexpr unsigned kMaxPlannedPairs = 4096;

__global__ __launch_bounds__(kThreads) void kv_load_counted_kernel(
    void* const* __restrict__ layers, size_t kv_stride, size_t block_bytes, unsigned num_blocks,
    const uint8_t* __restrict__ pool, uint64_t pool_blocks, size_t pool_block_bytes, unsigned store_first_layer,
    const int32_t* __restrict__ load_sel, unsigned n_slots, const int32_t* __restrict__ src_table, unsigned src_stride,
    const int32_t* __restrict__ dst_table, unsigned dst_stride, int64_t dst_layer_stride,
    const int32_t* __restrict__ load_count, const int32_t* __restrict__ rows, unsigned table_rows, unsigned batch,
    unsigned n_layers, StoredLayout lay)
{
    __shared__ unsigned s_total[kMaxPlannedPairs + 1];   // s_total[p] = loads of the pairs before p
    __shared__ unsigned s_part[kThreads];
    const unsigned pairs = n_layers * batch;             // pair p = layer p / batch, request p % batch
    constexpr unsigned kPer = kMaxPlannedPairs / kThreads;
    unsigned mine[kPer], sum = 0;
#pragma unroll
    for (unsigned i = 0; i < kPer; ++i) {
        const unsigned p = threadIdx.x * kPer + i;
        unsigned c = 0;
        if (p < pairs) {
            const unsigned l = p / batch, b = p - l * batch;
            const int32_t r = rows ? rows[b] : static_cast<int32_t>(b);
            if (r >= 0 && static_cast<unsigned>(r) < table_rows) {
                c = min(n_slots, static_cast<unsigned>(max(load_count[static_cast<size_t>(l) * table_rows + r], 0)));
            }
        }
        mine[i] = c;
        sum += c;
    }
    s_part[threadIdx.x] = sum;
    __syncthreads();
    for (unsigned d = 1; d < kThreads; d <<= 1) {         // inclusive scan of the threads' sums
        const unsigned v = threadIdx.x >= d ? s_part[threadIdx.x - d] : 0u;
        __syncthreads();
        s_part[threadIdx.x] += v;
        __syncthreads();
    }
    unsigned run = s_part[threadIdx.x] - sum;
#pragma unroll
    for (unsigned i = 0; i < kPer; ++i) {
        s_total[threadIdx.x * kPer + i] = run;
        run += mine[i];
    }
    if (threadIdx.x == kThreads - 1) { s_total[kMaxPlannedPairs] = run; }
    __syncthreads();
    const unsigned copies = 2u * s_total[kMaxPlannedPairs];
    for (unsigned w = blockIdx.x; w < copies; w += gridDim.x) {   // (uniform in the workgroup)
        const unsigned t = w >> 1, kv = w & 1u;
        unsigned lo = 0, hi = pairs;                     // last pair whose running total is <= t
        while (hi - lo > 1) {
            const unsigned mid = (lo + hi) >> 1;
            if (s_total[mid] <= t) { lo = mid; } else { hi = mid; }
        }
        const unsigned l = lo / batch, b = lo - l * batch, j = t - s_total[lo];
        const unsigned row = static_cast<unsigned>(rows ? rows[b] : static_cast<int32_t>(b));
        const int32_t sel = load_sel[(static_cast<size_t>(l) * table_rows + row) * n_slots + j];
        if (sel < 0 || static_cast<unsigned>(sel) >= src_stride) { continue; }
        const int32_t src = src_table[static_cast<size_t>(row) * src_stride + sel];
        if (src < 0 || static_cast<uint64_t>(src) >= pool_blocks) { continue; }
        const unsigned dst = static_cast<unsigned>(dst_table[l * dst_layer_stride + static_cast<int64_t>(row) * dst_stride + j]);
        if (dst >= num_blocks) { continue; }
        copy_slice(static_cast<uint8_t*>(layers[l]) + kv * kv_stride + static_cast<size_t>(dst) * block_bytes,
                   pool + static_cast<size_t>(src) * pool_block_bytes + lay.slice(store_first_layer + l, kv, block_bytes),
                   block_bytes);
    }
}

constexpr size_t kBatchPiece = 2 * kStep;  // 256 KiB

int check_block_args(const void* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                     int num_blocks, const void* ids, int n, const void* staging)
{
    UCM_REQUIRE(num_blocks > 0 && static_cast<size_t>(num_blocks) * block_bytes <= kv_stride,
                "kv move: num_blocks=%d does not fit kv_stride=%zu", num_blocks, kv_stride);
    UCM_REQUIRE(n == 0 || (layers && ids && staging), "kv move: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers <= 65535, "kv move: n_layers=%d out of range", n_layers);
    UCM_REQUIRE(n >= 0, "kv move: n=%d", n);
    UCM_REQUIRE(block_bytes > 0 && block_bytes % 16 == 0 && kv_stride % 16 == 0,
                "kv move: block_bytes=%zu / kv_stride=%zu must be multiples of 16", block_bytes, kv_stride);
    UCM_REQUIRE(ucm::aligned16(staging), "kv move: staging not 16-byte aligned");
    return UCM_OK;
}

int stored_layout(const char* name, size_t block_bytes, int rank, int tp_size, StoredLayout* lay)
{
    UCM_REQUIRE(tp_size >= 1 && rank >= 0 && rank < tp_size, "%s: rank=%d tp_size=%d", name, rank, tp_size);
    lay->layer_pitch = 2 * block_bytes * static_cast<size_t>(tp_size);
    lay->slice_base = 2 * block_bytes * static_cast<size_t>(rank);
    return UCM_OK;
}

// dst row dst_idx[i] = src row src_idx[i]: one 256-thread workgroup per pair (a step's query rows are a few KiB each,
// so the launch is all latency: every thread has its loads in flight before its first store)
constexpr int kRowThreads = 256;

__global__ __launch_bounds__(kRowThreads) void park_rows_kernel(const uint8_t* __restrict__ src, long long src_rows,
                                                                const int32_t* __restrict__ src_idx, uint8_t* __restrict__ dst,
                                                                long long dst_rows, const int32_t* __restrict__ dst_idx,
                                                                size_t row_bytes)
{
    const long long from = src_idx[blockIdx.x], to = dst_idx ? dst_idx[blockIdx.x] : static_cast<long long>(blockIdx.x);
    if (from < 0 || from >= src_rows || to < 0 || to >= dst_rows) { return; }
    const uint8_t* s = src + static_cast<size_t>(from) * row_bytes;
    uint8_t* d = dst + static_cast<size_t>(to) * row_bytes;
    for (size_t o = threadIdx.x * 16u; o < row_bytes; o += static_cast<size_t>(kRowThreads) * 16 * 4) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t at = o + static_cast<size_t>(u) * kRowThreads * 16;
            if (at < row_bytes) { v[u] = ucm::gload16(s + at); }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t at = o + static_cast<size_t>(u) * kRowThreads * 16;
            if (at < row_bytes) { ucm::gstore16(d + at, v[u]); }
        }
    }
}

}  // namespace

extern "C" int ucm_copy_batch(void* const* dst, const void* const* src, size_t num, size_t size,
                              ucm_stream_t stream)
{
    UCM_REQUIRE(size % 16 == 0, "ucm_copy_batch: size=%zu must be a multiple of 16", size);
    if (num == 0 || size == 0) { return UCM_OK; }
    UCM_REQUIRE(dst && src, "ucm_copy_batch: null pointer array");
    const size_t pieces = (size + kBatchPiece - 1) / kBatchPiece;
    UCM_REQUIRE(num * pieces <= 0x7fffffffull, "ucm_copy_batch: too many pieces for one launch");
    hipLaunchKernelGGL(copy_batch_kernel, dim3(static_cast<unsigned>(num * pieces)), dim3(kThreads), 0,
                       ucm::as_stream(stream), dst, src, size, kBatchPiece);
    UCM_LAUNCH_CHECK("ucm_copy_batch");
}

extern "C" int ucm_kv_gather_blocks_tp(const void* const* layers, int n_layers, size_t kv_stride,
                                       size_t block_bytes, int num_blocks, const int32_t* block_ids,
                                       int n, void* staging, int rank, int tp_size, ucm_stream_t stream)
{
    if (int rc = check_block_args(layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, staging)) { return rc; }
    StoredLayout lay;
    if (int rc = stored_layout("ucm_kv_gather_blocks", block_bytes, rank, tp_size, &lay)) { return rc; }
    if (n == 0) { return UCM_OK; }
    hipLaunchKernelGGL(kv_blocks_kernel<true>, dim3(static_cast<unsigned>(n), n_layers, 2),
                       dim3(kThreads), 0, ucm::as_stream(stream), const_cast<void* const*>(layers),
                       kv_stride, block_bytes, block_ids, static_cast<unsigned>(num_blocks),
                       static_cast<uint8_t*>(staging), lay);
    UCM_LAUNCH_CHECK("ucm_kv_gather_blocks");
}

extern "C" int ucm_kv_gather_blocks(const void* const* layers, int n_layers, size_t kv_stride,
                                    size_t block_bytes, int num_blocks, const int32_t* block_ids,
                                    int n, void* staging, ucm_stream_t stream)
{
    return ucm_kv_gather_blocks_tp(layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, staging, 0, 1, stream);
}

extern "C" int ucm_kv_scatter_blocks_tp(void* const* layers, int n_layers, size_t kv_stride,
                                        size_t block_bytes, int num_blocks, const int32_t* block_ids,
                                        int n, const void* staging, int rank, int tp_size, ucm_stream_t stream)
{
    if (int rc = check_block_args(layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, staging)) { return rc; }
    StoredLayout lay;
    if (int rc = stored_layout("ucm_kv_scatter_blocks", block_bytes, rank, tp_size, &lay)) { return rc; }
    if (n == 0) { return UCM_OK; }
    hipLaunchKernelGGL(kv_blocks_kernel<false>, dim3(static_cast<unsigned>(n), n_layers, 2),
                       dim3(kThreads), 0, ucm::as_stream(stream), layers, kv_stride, block_bytes,
                       block_ids, static_cast<unsigned>(num_blocks),
                       static_cast<uint8_t*>(const_cast<void*>(staging)), lay);
    UCM_LAUNCH_CHECK("ucm_kv_scatter_blocks");
}

extern "C" int ucm_kv_scatter_blocks(void* const* layers, int n_layers, size_t kv_stride,
                                     size_t block_bytes, int num_blocks, const int32_t* block_ids,
                                     int n, const void* staging, ucm_stream_t stream)
{
    return ucm_kv_scatter_blocks_tp(layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, staging, 0, 1, stream);
}

extern "C" int ucm_kv_gather_selected(const void* const* layers, int n_layers, size_t kv_stride,
                                      size_t block_bytes, int num_blocks, const int32_t* phys,
                                      const int32_t* count, int n_req, int phys_stride, const int64_t* dst_off,
                                      const int32_t* region_k, int max_count, void* staging,
                                      int64_t staging_blocks, ucm_stream_t stream)
{
    UCM_REQUIRE(staging_blocks >= 0, "ucm_kv_gather_selected: staging_blocks=%lld", static_cast<long long>(staging_blocks));
    UCM_REQUIRE(n_req == 0 || max_count == 0 || (layers && phys && count && dst_off && region_k && staging),
                "ucm_kv_gather_selected: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers * 2 <= 65535, "ucm_kv_gather_selected: n_layers=%d", n_layers);
    UCM_REQUIRE(num_blocks > 0 && static_cast<size_t>(num_blocks) * block_bytes <= kv_stride,
                "ucm_kv_gather_selected: num_blocks=%d does not fit kv_stride=%zu", num_blocks, kv_stride);
    UCM_REQUIRE(n_req >= 0 && n_req <= 65535, "ucm_kv_gather_selected: n_req=%d", n_req);
    UCM_REQUIRE(max_count >= 0 && phys_stride >= max_count,
                "ucm_kv_gather_selected: max_count=%d phys_stride=%d", max_count, phys_stride);
    UCM_REQUIRE(block_bytes > 0 && block_bytes % 16 == 0 && kv_stride % 16 == 0 && ucm::aligned16(staging),
                "ucm_kv_gather_selected: sizes and staging must be multiples of 16");
    if (n_req == 0 || max_count == 0) { return UCM_OK; }
    hipLaunchKernelGGL(kv_gather_selected_kernel,
                       dim3(static_cast<unsigned>(max_count), n_req, n_layers * 2),
                       dim3(kThreads), 0, ucm::as_stream(stream), layers, kv_stride, block_bytes, phys,
                       count, static_cast<unsigned>(num_blocks), static_cast<unsigned>(n_req), static_cast<unsigned>(phys_stride), dst_off,
                       region_k, static_cast<uint8_t*>(staging), static_cast<uint64_t>(staging_blocks));
    UCM_LAUNCH_CHECK("ucm_kv_gather_selected");
}

extern "C" int ucm_kv_load_planned_tp(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                                      int num_blocks, const void* pool, int64_t pool_blocks, size_t pool_block_bytes,
                                      int store_first_layer, const int32_t* load_sel, int n_slots,
                                      const int32_t* src_table, int src_stride, const int32_t* dst_table,
                                      int dst_stride, int64_t dst_layer_stride, const int32_t* load_count,
                                      const int32_t* rows, int batch, int table_rows, int rank, int tp_size,
                                      ucm_stream_t stream)
{
    StoredLayout lay;
    if (int rc = stored_layout("ucm_kv_load_planned", block_bytes, rank, tp_size, &lay)) { return rc; }
    UCM_REQUIRE(batch >= 0 && n_slots >= 0 && table_rows > 0, "ucm_kv_load_planned: batch=%d n_slots=%d table_rows=%d", batch,
                n_slots, table_rows);
    if (batch == 0 || n_slots == 0) { return UCM_OK; }
    UCM_REQUIRE(layers && pool && load_sel && src_table && dst_table, "ucm_kv_load_planned: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers * 2 <= 65535 && batch <= 65535, "ucm_kv_load_planned: n_layers=%d batch=%d", n_layers, batch);
    UCM_REQUIRE(num_blocks > 0 && static_cast<size_t>(num_blocks) * block_bytes <= kv_stride,
                "ucm_kv_load_planned: num_blocks=%d does not fit kv_stride=%zu", num_blocks, kv_stride);
    UCM_REQUIRE(block_bytes > 0 && block_bytes % 16 == 0 && kv_stride % 16 == 0 && pool_block_bytes % 16 == 0 &&
                    ucm::aligned16(pool),
                "ucm_kv_load_planned: sizes and pool must be multiples of 16");
    UCM_REQUIRE(store_first_layer >= 0 && pool_blocks >= 0 &&
                    static_cast<size_t>(store_first_layer + n_layers) * lay.layer_pitch <= pool_block_bytes,
                "ucm_kv_load_planned: layers %d..%d do not fit a stored block of %zu bytes", store_first_layer,
                store_first_layer + n_layers - 1, pool_block_bytes);
    UCM_REQUIRE(src_stride >= 1 && dst_stride >= n_slots && dst_layer_stride >= 0,
                "ucm_kv_load_planned: src_stride=%d dst_stride=%d n_slots=%d", src_stride, dst_stride, n_slots);
    if (load_count && static_cast<unsigned>(n_layers) * static_cast<unsigned>(batch) <= kMaxPlannedPairs) {
        // the rows' counts say exactly what there is to copy: 1024 workgroups share it evenly
        hipLaunchKernelGGL(kv_load_counted_kernel, dim3(1024), dim3(kThreads), 0, ucm::as_stream(stream), layers, kv_stride,
                           block_bytes, static_cast<unsigned>(num_blocks), static_cast<const uint8_t*>(pool),
                           static_cast<uint64_t>(pool_blocks), pool_block_bytes, static_cast<unsigned>(store_first_layer),
                           load_sel, static_cast<unsigned>(n_slots), src_table, static_cast<unsigned>(src_stride), dst_table,
                           static_cast<unsigned>(dst_stride), dst_layer_stride, load_count, rows,
                           static_cast<unsigned>(table_rows), static_cast<unsigned>(batch), static_cast<unsigned>(n_layers), lay);
    } else {
        // the entries to load are scattered over a row (or there are too many rows for the counted kernel's table)
        // A small launch (one layer's plan for a batch) takes a workgroup per slot: the slots that load are scattered,
        // and with 16 workgroups stepping through a row some copy three blocks while others copy none (a layer of 16
        // requests with 40 % of 48 slots to load: 190 us stepping, about as long as loading all of them).  A big one (every
        // layer's plan in one launch) keeps the stepping: there the workgroups that find nothing are the many.
        const int64_t per_slot = static_cast<int64_t>(n_slots) * batch * n_layers * 2;
        const unsigned gx = static_cast<unsigned>(per_slot <= 8192 ? n_slots : std::min(n_slots, load_count ? 8 : 16));
        hipLaunchKernelGGL(kv_load_planned_kernel, dim3(gx, batch, n_layers * 2), dim3(kThreads), 0,
                           ucm::as_stream(stream), layers, kv_stride, block_bytes, static_cast<unsigned>(num_blocks),
                           static_cast<const uint8_t*>(pool), static_cast<uint64_t>(pool_blocks), pool_block_bytes,
                           static_cast<unsigned>(store_first_layer), load_sel, static_cast<unsigned>(n_slots), src_table,
                           static_cast<unsigned>(src_stride), dst_table, static_cast<unsigned>(dst_stride), dst_layer_stride,
                           load_count, rows, static_cast<unsigned>(table_rows), lay);
    }
    UCM_LAUNCH_CHECK("ucm_kv_load_planned");
}

extern "C" int ucm_kv_load_planned(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                                   int num_blocks, const void* pool, int64_t pool_blocks, size_t pool_block_bytes,
                                   int store_first_layer, const int32_t* load_sel, int n_slots,
                                   const int32_t* src_table, int src_stride, const int32_t* dst_table,
                                   int dst_stride, int64_t dst_layer_stride, const int32_t* load_count,
                                   const int32_t* rows, int batch, int table_rows, ucm_stream_t stream)
{
    return ucm_kv_load_planned_tp(layers, n_layers, kv_stride, block_bytes, num_blocks, pool, pool_blocks, pool_block_bytes,
                                  store_first_layer, load_sel, n_slots, src_table, src_stride, dst_table, dst_stride,
                                  dst_layer_stride, load_count, rows, batch, table_rows, 0, 1, stream);
}

extern "C" int ucm_park_rows(const void* src, int64_t src_rows, const int32_t* src_idx, void* dst, int64_t dst_rows,
                             const int32_t* dst_idx, int n, size_t row_bytes, ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0 && src_rows >= 0 && dst_rows >= 0, "ucm_park_rows: n=%d src_rows=%lld dst_rows=%lld", n,
                static_cast<long long>(src_rows), static_cast<long long>(dst_rows));
    UCM_REQUIRE(row_bytes > 0 && row_bytes % 16 == 0, "ucm_park_rows: row_bytes=%zu must be a positive multiple of 16", row_bytes);
    if (n == 0) { return UCM_OK; }
    UCM_REQUIRE(src && src_idx && dst, "ucm_park_rows: null pointer");
    UCM_REQUIRE(ucm::aligned16(src) && ucm::aligned16(dst), "ucm_park_rows: src and dst must be 16-byte aligned");
    hipLaunchKernelGGL(park_rows_kernel, dim3(static_cast<unsigned>(n)), dim3(kRowThreads), 0, ucm::as_stream(stream),
                       static_cast<const uint8_t*>(src), static_cast<long long>(src_rows), src_idx, static_cast<uint8_t*>(dst),
                       static_cast<long long>(dst_rows), dst_idx, row_bytes);
    UCM_LAUNCH_CHECK("ucm_park_rows");
}
