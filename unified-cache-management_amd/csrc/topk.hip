// Per-request block selection with forced windows: one 64-wide wavefront per
// (layer, request); the selection itself is ucm::select_wave (topk_select.h).
//
// A few KB in, a few hundred bytes out per wave: this kernel is latency-bound,
// not bandwidth-bound; it only has to stay small next to scoring and gather.
#include "common.h"
#include "topk_select.h"

namespace {

using ucm::lanes_below;
using ucm::ordered_key;

// grid: x = request, y = layer; block = one wave
template <int kEpl, bool kHeapTies>
__global__ __launch_bounds__(64) void topk_windows_kernel(const ucm::SelectArgs a)
{
    ucm::select_wave<kEpl, kHeapTies>(a, blockIdx.x, blockIdx.y, threadIdx.x);
}

template <bool kHeapTies>
void launch_select(const ucm::SelectArgs& a, int max_seg_len, int n_layers, hipStream_t s)
{
    const dim3 grid(a.n_req, n_layers), block(64);
#define UCM_TOPK_LAUNCH(EPL) hipLaunchKernelGGL((topk_windows_kernel<EPL, kHeapTies>), grid, block, 0, s, a)
    // registers per lane for the keys: the smallest tier that holds the longest request (the radix steps cost
    // one ballot per register and bit)
    if (max_seg_len <= 64) { UCM_TOPK_LAUNCH(1); }
    else if (max_seg_len <= 128) { UCM_TOPK_LAUNCH(2); }
    else if (max_seg_len <= 256) { UCM_TOPK_LAUNCH(4); }
    else if (max_seg_len <= 512) { UCM_TOPK_LAUNCH(8); }
    else if (max_seg_len <= 1024) { UCM_TOPK_LAUNCH(16); }
    else if (max_seg_len <= 2048) { UCM_TOPK_LAUNCH(32); }
    else { UCM_TOPK_LAUNCH(64); }
#undef UCM_TOPK_LAUNCH
}

}  // namespace

extern "C" int ucm_topk_windows(const float* scores, int64_t scores_layer_stride, int64_t scores_rows,
                                const int32_t* seg_off, const int32_t* seg_len, const int32_t* topk_len, int n_req,
                                int max_seg_len, int n_layers, int start_w, int end_w, int32_t* idx_out,
                                int out_stride, int32_t* count_out, const int32_t* block_tables, int bt_stride,
                                int32_t* phys_out, const int32_t* seq_lens, int block_size,
                                int32_t* sparse_seq_lens, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req == 0 || (scores && seg_off && seg_len && topk_len && idx_out && count_out),
                "ucm_topk_windows: null pointer");
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535, "ucm_topk_windows: n_req=%d n_layers=%d", n_req, n_layers);
    UCM_REQUIRE(start_w >= 0 && end_w >= 0 && max_seg_len >= 0, "ucm_topk_windows: negative window or length");
    UCM_REQUIRE(scores_rows >= 0 && (n_layers == 1 || scores_layer_stride >= scores_rows),
                "ucm_topk_windows: scores_rows=%lld does not fit scores_layer_stride=%lld",
                static_cast<long long>(scores_rows), static_cast<long long>(scores_layer_stride));
    UCM_REQUIRE(out_stride >= max_seg_len, "ucm_topk_windows: out_stride=%d < max_seg_len=%d", out_stride, max_seg_len);
    UCM_REQUIRE((block_tables == nullptr) == (phys_out == nullptr),
                "ucm_topk_windows: block_tables and phys_out go together");
    UCM_REQUIRE(!block_tables || bt_stride >= max_seg_len, "ucm_topk_windows: bt_stride=%d < max_seg_len=%d",
                bt_stride, max_seg_len);
    UCM_REQUIRE(!sparse_seq_lens || (seq_lens && block_size > 0), "ucm_topk_windows: sparse_seq_lens needs seq_lens and block_size");
    UCM_SUPPORTED(max_seg_len <= 4096, "ucm_topk_windows: max_seg_len=%d (at most 4096 blocks per request)", max_seg_len);
    if (n_req == 0) { return UCM_OK; }
    const ucm::SelectArgs a = {scores, scores_layer_stride, scores_rows, seg_off, seg_len, topk_len, n_req, max_seg_len,
                               start_w, end_w, idx_out, out_stride, static_cast<int64_t>(n_req) * out_stride, n_req, count_out, block_tables, bt_stride, phys_out, seq_lens, block_size,
                               sparse_seq_lens};
    launch_select<false>(a, max_seg_len, n_layers, ucm::as_stream(stream));
    UCM_LAUNCH_CHECK("ucm_topk_windows");
}

extern "C" int ucm_kvstar_topk(const float* votes, int64_t votes_rows, const int32_t* seg_off, const int32_t* seg_len,
                               const int32_t* topk_len, int n_tasks, int max_seg_len, int32_t* idx_out,
                               int out_stride, int32_t* count_out, ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks >= 0 && max_seg_len >= 0 && votes_rows >= 0, "ucm_kvstar_topk: n_tasks=%d max_seg_len=%d votes_rows=%lld",
                n_tasks, max_seg_len, static_cast<long long>(votes_rows));
    if (n_tasks == 0) { return UCM_OK; }
    UCM_REQUIRE(votes && seg_off && seg_len && topk_len && idx_out && count_out, "ucm_kvstar_topk: null pointer");
    UCM_REQUIRE(out_stride >= max_seg_len, "ucm_kvstar_topk: out_stride=%d < max_seg_len=%d", out_stride, max_seg_len);
    UCM_SUPPORTED(max_seg_len <= 4096, "ucm_kvstar_topk: max_seg_len=%d (at most 4096 blocks per task)", max_seg_len);
    const ucm::SelectArgs a = {votes, 0, votes_rows, seg_off, seg_len, topk_len, n_tasks, max_seg_len, 0, 0, idx_out, out_stride, 0, 0, count_out,
                               nullptr, 0, nullptr, nullptr, 1, nullptr};
    launch_select<true>(a, max_seg_len, 1, ucm::as_stream(stream));
    UCM_LAUNCH_CHECK("ucm_kvstar_topk");
}

// ---------------------------------------------------------------------------
// The order KVStar's heap hands its pairs back in (descending by (score, index),
// simd_compute_kernel.cpp:969-977), restored on the device: a task's chosen blocks are ranked by counting - the
// 64-bit keys (ordered score, index) are distinct, so entry j goes to position #{m : key[m] > key[j]}.  One
// workgroup per task, the keys in LDS, every thread reading the same key at a time (a broadcast).
namespace {

constexpr int kOrderThreads = 256;
constexpr int kOrderMax = 4096;

__global__ __launch_bounds__(kOrderThreads) void kvstar_order_kernel(
    const float* __restrict__ votes, int64_t votes_rows, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, int32_t* __restrict__ idx, int out_stride, const int32_t* __restrict__ count)
{
    __shared__ unsigned long long keys[kOrderMax];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int n = seg_len[t];
    const int64_t seg0 = seg_off[t];
    // a task whose votes lie outside the array is left as it is (the selection wrote nothing for it either)
    if (seg0 < 0 || n < 0 || seg0 + n > votes_rows) { return; }
    const int k = min(count[t], min(out_stride, kOrderMax));
    int32_t* row = idx + static_cast<size_t>(t) * out_stride;
    const float* v = votes + seg0;
    for (int j = tid; j < k; j += kOrderThreads) {
        const int i = row[j];
        const bool inside = i >= 0 && i < n;             // anything else was not written by the selection: never read
        keys[j] = (static_cast<unsigned long long>(inside ? ordered_key(v[i]) : 0u) << 32) | static_cast<unsigned>(i);
    }
    __syncthreads();
    for (int j = tid; j < k; j += kOrderThreads) {
        const unsigned long long mine = keys[j];
        int rank = 0;
        for (int m = 0; m < k; ++m) { rank += keys[m] > mine ? 1 : 0; }
        row[rank] = static_cast<int32_t>(static_cast<unsigned>(mine));
    }
}

}  // namespace

extern "C" int ucm_kvstar_order(const float* votes, int64_t votes_rows, const int32_t* seg_off, const int32_t* seg_len,
                                int n_tasks, int max_count, int32_t* idx_io, int out_stride, const int32_t* count,
                                ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks >= 0 && max_count >= 0 && votes_rows >= 0, "ucm_kvstar_order: n_tasks=%d max_count=%d votes_rows=%lld",
                n_tasks, max_count, static_cast<long long>(votes_rows));
    if (n_tasks == 0 || max_count == 0) { return UCM_OK; }
    UCM_REQUIRE(votes && seg_off && seg_len && idx_io && count, "ucm_kvstar_order: null pointer");
    UCM_REQUIRE(out_stride >= max_count, "ucm_kvstar_order: out_stride=%d < max_count=%d", out_stride, max_count);
    UCM_SUPPORTED(max_count <= kOrderMax, "ucm_kvstar_order: max_count=%d (at most 4096 chosen blocks per task)", max_count);
    hipLaunchKernelGGL(kvstar_order_kernel, dim3(n_tasks), dim3(kOrderThreads), 0, ucm::as_stream(stream), votes,
                       votes_rows, seg_off, seg_len, idx_io, out_stride, count);
    UCM_LAUNCH_CHECK("ucm_kvstar_order");
}

// ---------------------------------------------------------------------------
// Resident-set bookkeeping for delta loads: which of a request's staging slots
// already hold a block of the new selection, and which missing block goes to
// which freed slot.  One wave per (layer, request), slot j and selection entry
// j in lane j; membership is a k-step broadcast compare, ranks are ballot
// prefix counts, so the i-th missing block (ascending) lands in the i-th freed
// slot (ascending) - a deterministic refinement of the reference's set
// arithmetic (ucm/sparse/esa/esa.py:312-338).
namespace {

// grid: x = request, y = layer; block = one wave; n_slots <= 64
__global__ __launch_bounds__(64) void delta_plan_kernel(
    const int32_t* __restrict__ sel, const int32_t* __restrict__ sel_phys, const int32_t* __restrict__ count,
    int n_req, int sel_stride, int32_t* __restrict__ resident, int n_slots, int32_t* __restrict__ load_phys,
    int32_t* __restrict__ slot_of_sel, int32_t* __restrict__ miss_count, const int32_t* __restrict__ rows)
{
    const int l = blockIdx.y, lane = threadIdx.x;
    int r = blockIdx.x;
    if (rows) {   // a call over some rows of a persistent request table of n_req rows
        r = rows[r];
        if (r < 0 || r >= n_req) { return; }
    }
    const size_t lr = static_cast<size_t>(l) * n_req + r;
    const int k = min(min(count[lr], n_slots), sel_stride);   // selections beyond the slot budget cannot be resident
    const int32_t* s = sel + lr * sel_stride;
    const int32_t* sp = sel_phys + lr * sel_stride;
    int32_t* res = resident + lr * n_slots;

    const int my_sel = lane < k ? s[lane] : -1;
    const int my_phys = lane < k ? sp[lane] : -1;
    const int my_res = lane < n_slots ? res[lane] : -1;

    // selection entry `lane` already resident?  slot `lane` still wanted?
    bool hit = false, keep = false;
    int hit_slot = -1;
    for (int j = 0; j < 64; ++j) {
        const int rj = __shfl(my_res, j, 64);
        const int sj = __shfl(my_sel, j, 64);
        if (j < n_slots && rj >= 0 && rj == my_sel && my_sel >= 0) { hit = true; hit_slot = j; }
        if (j < k && sj >= 0 && sj == my_res && my_res >= 0) { keep = true; }
    }
    const bool miss = lane < k && !hit;
    const bool freed = lane < n_slots && !keep;
    const unsigned long long miss_mask = __ballot(miss), free_mask = __ballot(freed);
    const int miss_rank = static_cast<int>(lanes_below(miss_mask));
    const int free_rank = static_cast<int>(lanes_below(free_mask));

    // the slot with free rank q receives the miss with miss rank q (exchanged through LDS)
    __shared__ int32_t miss_sel[64], miss_phys[64], free_slot[64];
    if (miss) { miss_sel[miss_rank] = my_sel; miss_phys[miss_rank] = my_phys; }
    if (freed) { free_slot[free_rank] = lane; }
    __syncthreads();
    const int n_move = min(__popcll(miss_mask), __popcll(free_mask));
    int dst_slot = hit_slot;
    int take_sel = -1, take_phys = -1;
    if (freed && free_rank < n_move) { take_sel = miss_sel[free_rank]; take_phys = miss_phys[free_rank]; }
    if (miss && miss_rank < n_move) { dst_slot = free_slot[miss_rank]; }
    if (lane < n_slots) {
        load_phys[lr * n_slots + lane] = take_phys;              // -1: slot keeps what it holds
        if (take_sel >= 0) { res[lane] = take_sel; }
        else if (freed) { res[lane] = -1; }                      // block dropped, nothing to replace it
    }
    if (lane < k) { slot_of_sel[lr * sel_stride + lane] = dst_slot; }
    if (lane == 0) { miss_count[lr] = n_move; }
}

// More than 64 slots: one 256-thread workgroup per (layer, request), entry
// e*256 + thread in register e.  Both lists sit in LDS and every thread walks
// the other list four entries per read (all threads read the same address, a
// broadcast); ranks are ballot prefix counts plus the counts of the (register,
// wave) groups before the thread's own, so the pairing is the same as above.
constexpr int kPlanThreads = 256;
constexpr int kPlanWaves = kPlanThreads / 64;

template <int E>  // entries per thread: n_slots <= 256 * E
__global__ __launch_bounds__(kPlanThreads) void delta_plan_wide_kernel(
    const int32_t* __restrict__ sel, const int32_t* __restrict__ sel_phys, const int32_t* __restrict__ count,
    int n_req, int sel_stride, int32_t* __restrict__ resident, int n_slots, int32_t* __restrict__ load_phys,
    int32_t* __restrict__ slot_of_sel, int32_t* __restrict__ miss_count, const int32_t* __restrict__ rows)
{
    constexpr int kCap = kPlanThreads * E;
    const int l = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    int r = blockIdx.x;
    if (rows) {
        r = rows[r];
        if (r < 0 || r >= n_req) { return; }
    }
    const size_t lr = static_cast<size_t>(l) * n_req + r;
    const int k = min(min(count[lr], n_slots), sel_stride);   // (a count larger than a row of sel is never followed)
    const int32_t* s = sel + lr * sel_stride;
    const int32_t* sp = sel_phys + lr * sel_stride;
    int32_t* res = resident + lr * n_slots;

    __shared__ __attribute__((aligned(16))) int32_t s_sel[kCap], s_res[kCap];
    __shared__ int32_t s_a[kCap], s_b[kCap], s_c[kCap];   // miss_sel, miss_phys, free_slot by rank
    __shared__ int s_miss_cnt[E * kPlanWaves], s_free_cnt[E * kPlanWaves];

    int my_sel[E], my_phys[E], my_res[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int i = e * kPlanThreads + tid;
        my_sel[e] = i < k ? s[i] : -1;
        my_phys[e] = i < k ? sp[i] : -1;
        my_res[e] = i < n_slots ? res[i] : -1;
        s_sel[i] = my_sel[e];          // entries past the lists hold -1, which matches nothing
        s_res[i] = my_res[e];
    }
    __syncthreads();

    int hit_slot[E];
    bool keep[E];
#pragma unroll
    for (int e = 0; e < E; ++e) { hit_slot[e] = -1; keep[e] = false; }
    const int res_quads = (n_slots + 3) >> 2, sel_quads = (k + 3) >> 2;
    for (int q = 0; q < res_quads; ++q) {
        const int4 v = *reinterpret_cast<const int4*>(&s_res[q * 4]);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if (my_sel[e] >= 0) {   // the last matching slot wins, as in the one-wave kernel
                if (v.x == my_sel[e]) { hit_slot[e] = q * 4; }
                if (v.y == my_sel[e]) { hit_slot[e] = q * 4 + 1; }
                if (v.z == my_sel[e]) { hit_slot[e] = q * 4 + 2; }
                if (v.w == my_sel[e]) { hit_slot[e] = q * 4 + 3; }
            }
        }
    }
    for (int q = 0; q < sel_quads; ++q) {
        const int4 v = *reinterpret_cast<const int4*>(&s_sel[q * 4]);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if (my_res[e] >= 0 && (v.x == my_res[e] || v.y == my_res[e] || v.z == my_res[e] || v.w == my_res[e])) {
                keep[e] = true;
            }
        }
    }

    bool miss[E], freed[E];
    int miss_rank[E], free_rank[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int i = e * kPlanThreads + tid;
        miss[e] = i < k && hit_slot[e] < 0;
        freed[e] = i < n_slots && !keep[e];
        const unsigned long long mm = __ballot(miss[e]), fm = __ballot(freed[e]);
        miss_rank[e] = static_cast<int>(lanes_below(mm));
        free_rank[e] = static_cast<int>(lanes_below(fm));
        if (lane == 0) { s_miss_cnt[e * kPlanWaves + wave] = __popcll(mm); s_free_cnt[e * kPlanWaves + wave] = __popcll(fm); }
    }
    __syncthreads();
    int n_miss = 0, n_free = 0;
#pragma unroll
    for (int g = 0; g < E * kPlanWaves; ++g) {
        const int cm = s_miss_cnt[g], cf = s_free_cnt[g];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if (g < e * kPlanWaves + wave) { miss_rank[e] += cm; free_rank[e] += cf; }
        }
        n_miss += cm;
        n_free += cf;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
        if (miss[e]) { s_a[miss_rank[e]] = my_sel[e]; s_b[miss_rank[e]] = my_phys[e]; }
        if (freed[e]) { s_c[free_rank[e]] = e * kPlanThreads + tid; }
    }
    __syncthreads();
    const int n_move = min(n_miss, n_free);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int i = e * kPlanThreads + tid;
        int dst_slot = hit_slot[e], take_sel = -1, take_phys = -1;
        if (freed[e] && free_rank[e] < n_move) { take_sel = s_a[free_rank[e]]; take_phys = s_b[free_rank[e]]; }
        if (miss[e] && miss_rank[e] < n_move) { dst_slot = s_c[miss_rank[e]]; }
        if (i < n_slots) {
            load_phys[lr * n_slots + i] = take_phys;
            if (take_sel >= 0) { res[i] = take_sel; }
            else if (freed[e]) { res[i] = -1; }
        }
        if (i < k) { slot_of_sel[lr * sel_stride + i] = dst_slot; }
    }
    if (tid == 0) { miss_count[lr] = n_move; }
}

}  // namespace

namespace {

int delta_plan_launch(const char* name, const int32_t* sel, const int32_t* sel_phys, const int32_t* count, int n_rows,
                      int n_launch, const int32_t* rows, int n_layers, int sel_stride, int32_t* resident, int n_slots,
                      int32_t* load_phys, int32_t* slot_of_sel, int32_t* miss_count, ucm_stream_t stream)
{
    const dim3 grid(n_launch, n_layers);
    hipStream_t s = ucm::as_stream(stream);
#define UCM_PLAN_LAUNCH(E)                                                                                    \
    hipLaunchKernelGGL(delta_plan_wide_kernel<E>, grid, dim3(kPlanThreads), 0, s, sel, sel_phys, count, n_rows, \
                       sel_stride, resident, n_slots, load_phys, slot_of_sel, miss_count, rows)
    if (n_slots <= 64) {
        hipLaunchKernelGGL(delta_plan_kernel, grid, dim3(64), 0, s, sel, sel_phys, count, n_rows, sel_stride, resident,
                           n_slots, load_phys, slot_of_sel, miss_count, rows);
    }
    else if (n_slots <= 256) { UCM_PLAN_LAUNCH(1); }
    else if (n_slots <= 512) { UCM_PLAN_LAUNCH(2); }
    else { UCM_PLAN_LAUNCH(4); }
#undef UCM_PLAN_LAUNCH
    return ucm::check_hip(hipGetLastError(), name);
}

}  // namespace

extern "C" int ucm_delta_plan(const int32_t* sel, const int32_t* sel_phys, const int32_t* count, int n_req,
                              int n_layers, int sel_stride, int32_t* resident, int n_slots, int32_t* load_phys,
                              int32_t* slot_of_sel, int32_t* miss_count, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535, "ucm_delta_plan: n_req=%d n_layers=%d", n_req, n_layers);
    if (n_req == 0) { return UCM_OK; }
    UCM_REQUIRE(sel && sel_phys && count && resident && load_phys && slot_of_sel && miss_count, "ucm_delta_plan: null pointer");
    UCM_SUPPORTED(n_slots >= 1 && n_slots <= 1024, "ucm_delta_plan: n_slots=%d (1..1024 staging slots per request and layer)", n_slots);
    UCM_REQUIRE(sel_stride >= 1, "ucm_delta_plan: sel_stride=%d", sel_stride);
    return delta_plan_launch("ucm_delta_plan", sel, sel_phys, count, n_req, n_req, nullptr, n_layers, sel_stride, resident,
                             n_slots, load_phys, slot_of_sel, miss_count, stream);
}

extern "C" int ucm_delta_plan_rows(const int32_t* sel, const int32_t* sel_phys, const int32_t* count,
                                   const int32_t* rows, int batch, int table_rows, int n_layers, int sel_stride,
                                   int32_t* resident, int n_slots, int32_t* load_phys, int32_t* slot_of_sel,
                                   int32_t* miss_count, ucm_stream_t stream)
{
    UCM_REQUIRE(batch >= 0 && table_rows > 0 && n_layers > 0 && n_layers <= 65535,
                "ucm_delta_plan_rows: batch=%d table_rows=%d n_layers=%d", batch, table_rows, n_layers);
    if (batch == 0) { return UCM_OK; }
    UCM_REQUIRE(sel && sel_phys && count && rows && resident && load_phys && slot_of_sel && miss_count,
                "ucm_delta_plan_rows: null pointer");
    UCM_SUPPORTED(n_slots >= 1 && n_slots <= 1024, "ucm_delta_plan_rows: n_slots=%d (1..1024 staging slots per request and layer)", n_slots);
    UCM_REQUIRE(sel_stride >= 1, "ucm_delta_plan_rows: sel_stride=%d", sel_stride);
    return delta_plan_launch("ucm_delta_plan_rows", sel, sel_phys, count, table_rows, batch, rows, n_layers, sel_stride,
                             resident, n_slots, load_phys, slot_of_sel, miss_count, stream);
}
