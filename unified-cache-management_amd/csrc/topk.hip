// Per-request block selection with forced windows: one 64-wide wavefront per
// (layer, request), the request's scores held in registers as order-preserving
// 32-bit keys (element i lives in lane i%64, register i/64).
//
// Selection is a radix select, one bit per step from the top: the threshold T
// is grown greedily while at least m candidates have key >= T, each count being
// a wave ballot + popcount.  Candidates with key > T are all taken; of those
// with key == T the first `m - count(key > T)` in index order are taken, which
// is exactly where a stable descending sort leaves equal scores.  Output
// positions are ballot prefix counts in index order, so the result comes out
// sorted ascending with no sort at all, and the logical->physical block-table
// lookup is applied on the way out.
//
// A few KB in, a few hundred bytes out per wave: this kernel is latency-bound,
// not bandwidth-bound; it only has to stay small next to scoring and gather.
#include "common.h"

namespace {

__device__ __forceinline__ unsigned ordered_key(float f)
{
    f = f + 0.0f;  // -0.0 -> +0.0, so that the two zeros tie like they do under operator>
    const unsigned u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ unsigned lanes_below(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u));
}

// kHeapTies selects which blocks tied at the k-th score are kept.  false: the
// first ones in index order (std::stable_sort).  true: the ones KVStar's
// min-heap of (score, index) pairs ends up with
// (ucm/sparse/kvstar/retrieve/core/domain/retrieve_task/simd_compute_kernel.cpp:955-977:
// blocks arrive in index order, a full heap replaces its smallest pair only
// for a strictly greater score).  That process has a closed form: ties enter
// while fewer than k blocks with key >= T have arrived and leave, lowest index
// first, once per block above T that arrives later; so with P the shortest
// prefix holding k blocks >= T, g_P the blocks above T inside P and g those in
// the whole list, the ties kept are the ones of P whose rank among the ties is
// at least g - g_P.  Windows are not used with it (host checked).
//
// grid: x = request, y = layer; block = one wave
template <int kEpl, bool kHeapTies>
__global__ __launch_bounds__(64) void topk_windows_kernel(
    const float* __restrict__ scores, int64_t scores_layer_stride, const int32_t* __restrict__ seg_off,
    const int32_t* __restrict__ seg_len, const int32_t* __restrict__ topk_len, int n_req, int start_w,
    int end_w, int32_t* __restrict__ idx_out, int out_stride, int32_t* __restrict__ count_out,
    const int32_t* __restrict__ block_tables, int bt_stride, int32_t* __restrict__ phys_out,
    const int32_t* __restrict__ seq_lens, int block_size, int32_t* __restrict__ sparse_seq_lens)
{
    const int r = blockIdx.x, l = blockIdx.y, lane = threadIdx.x;
    const size_t lr = static_cast<size_t>(l) * n_req + r;
    int n = seg_len[r];
    n = min(n, min(out_stride, 64 * kEpl));  // host checked; clamp so nothing can run past a row
    if (block_tables) { n = min(n, bt_stride); }
    const int k = topk_len[r];
    int32_t* out = idx_out + lr * out_stride;
    int32_t* pout = phys_out ? phys_out + lr * out_stride : nullptr;
    const int32_t* bt = block_tables ? block_tables + static_cast<size_t>(r) * bt_stride : nullptr;
    int count = 0;
    bool kept_all = false;

    if (n <= 0) {
        count = 0;
    } else if (start_w + end_w >= n || k >= n || k <= 0) {
        for (int i = lane; i < n; i += 64) {
            out[i] = i;
            if (pout) { pout[i] = bt[i]; }
        }
        count = n;
        kept_all = true;
    } else if (k < start_w + end_w) {
        // fewer slots than forced blocks: the first k of [0..start_w) ++ [n-end_w..n)
        for (int j = lane; j < k; j += 64) {
            const int idx = j < start_w ? j : n - end_w + (j - start_w);
            out[j] = idx;
            if (pout) { pout[j] = bt[idx]; }
        }
        count = k;
    } else {
        const int m = k - start_w - end_w;       // free picks among the middle blocks
        const int hi = n - end_w;                // candidates are start_w <= i < hi
        const float* s = scores + static_cast<int64_t>(l) * scores_layer_stride + seg_off[r];
        unsigned key[kEpl];
        int32_t phys[kEpl];                      // the block table's entries, fetched with the scores: a load per
#pragma unroll                                   // taken element on the way out would cost a memory round trip per register
        for (int j = 0; j < kEpl; ++j) {
            const int i = j * 64 + lane;
            const bool cand = i >= start_w && i < hi;
            key[j] = cand ? ordered_key(s[cand ? i : 0]) : 0u;
            phys[j] = bt ? bt[min(i, n - 1)] : 0;
        }
        unsigned T = 0;
        int need = 0;
        int tie_lo = 0, tie_hi = 0;              // kHeapTies: ranks (among the ties) that are kept
        if (m > 0) {
            for (int bit = 31; bit >= 0; --bit) {
                const unsigned c = T | (1u << bit);
                int cnt = 0;
#pragma unroll
                for (int j = 0; j < kEpl; ++j) { cnt += __popcll(__ballot(key[j] >= c)); }
                if (cnt >= m) { T = c; }
            }
            int greater = 0;
#pragma unroll
            for (int j = 0; j < kEpl; ++j) { greater += __popcll(__ballot(key[j] > T)); }
            need = m - greater;
            if (kHeapTies) {
                // walk the list in index order up to the k-th block with key >= T
                int seen = 0, g_p = 0;
#pragma unroll
                for (int j = 0; j < kEpl; ++j) {
                    const unsigned long long ge_mask = __ballot(key[j] >= T && key[j] != 0u);
                    const unsigned long long gt_mask = __ballot(key[j] > T);
                    const int c = __popcll(ge_mask);
                    if (seen < m) {
                        if (seen + c >= m) {
                            // lane holding the m-th one: the (m - seen)-th set bit of ge_mask
                            const bool is_pth = ((ge_mask >> lane) & 1ull) && seen + static_cast<int>(lanes_below(ge_mask)) + 1 == m;
                            const unsigned long long pm = __ballot(is_pth);
                            const int p_lane = __ffsll(static_cast<long long>(pm)) - 1;
                            const unsigned long long upto = p_lane >= 63 ? ~0ull : ((2ull << p_lane) - 1ull);
                            g_p += __popcll(gt_mask & upto);
                        } else {
                            g_p += __popcll(gt_mask);
                        }
                    }
                    seen += c;
                }
                tie_lo = greater - g_p;          // one tie left per block above T that came after P
                tie_hi = m - g_p;                // ties inside P
            }
        }
        int pos = 0, ties_seen = 0;
#pragma unroll
        for (int j = 0; j < kEpl; ++j) {
            if (j * 64 < n) {
                const int i = j * 64 + lane;
                const bool window = i < n && (i < start_w || i >= hi);
                const bool cand = i >= start_w && i < hi;
                const bool gt = cand && m > 0 && key[j] > T;
                const bool eq = cand && m > 0 && key[j] == T;
                const unsigned long long eq_mask = __ballot(eq);
                const int tie_rank = ties_seen + static_cast<int>(lanes_below(eq_mask));
                const bool take = window || gt || (eq && (kHeapTies ? (tie_rank >= tie_lo && tie_rank < tie_hi) : tie_rank < need));
                ties_seen += __popcll(eq_mask);
                const unsigned long long take_mask = __ballot(take);
                if (take) {
                    const int p = pos + static_cast<int>(lanes_below(take_mask));
                    out[p] = i;
                    if (pout) { pout[p] = phys[j]; }
                }
                pos += __popcll(take_mask);
            }
        }
        count = pos;
    }
    if (lane == 0) {
        count_out[lr] = count;
        if (sparse_seq_lens && seq_lens) {
            const int len = seq_lens[r], rem = len % block_size;
            // every block kept: the request keeps its length; otherwise `count` blocks, the last one partial
            sparse_seq_lens[lr] = kept_all ? len : (rem == 0 ? count * block_size : count * block_size - block_size + rem);
        }
    }
}

}  // namespace

extern "C" int ucm_topk_windows(const float* scores, int64_t scores_layer_stride, const int32_t* seg_off,
                                const int32_t* seg_len, const int32_t* topk_len, int n_req, int max_seg_len,
                                int n_layers, int start_w, int end_w, int32_t* idx_out, int out_stride,
                                int32_t* count_out, const int32_t* block_tables, int bt_stride,
                                int32_t* phys_out, const int32_t* seq_lens, int block_size,
                                int32_t* sparse_seq_lens, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req == 0 || (scores && seg_off && seg_len && topk_len && idx_out && count_out),
                "ucm_topk_windows: null pointer");
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535, "ucm_topk_windows: n_req=%d n_layers=%d", n_req, n_layers);
    UCM_REQUIRE(start_w >= 0 && end_w >= 0 && max_seg_len >= 0, "ucm_topk_windows: negative window or length");
    UCM_REQUIRE(out_stride >= max_seg_len, "ucm_topk_windows: out_stride=%d < max_seg_len=%d", out_stride, max_seg_len);
    UCM_REQUIRE((block_tables == nullptr) == (phys_out == nullptr),
                "ucm_topk_windows: block_tables and phys_out go together");
    UCM_REQUIRE(!block_tables || bt_stride >= max_seg_len, "ucm_topk_windows: bt_stride=%d < max_seg_len=%d",
                bt_stride, max_seg_len);
    UCM_REQUIRE(!sparse_seq_lens || (seq_lens && block_size > 0), "ucm_topk_windows: sparse_seq_lens needs seq_lens and block_size");
    UCM_SUPPORTED(max_seg_len <= 4096, "ucm_topk_windows: max_seg_len=%d (at most 4096 blocks per request)", max_seg_len);
    if (n_req == 0) { return UCM_OK; }
    hipStream_t s = ucm::as_stream(stream);
    const dim3 grid(n_req, n_layers), block(64);
#define UCM_TOPK_LAUNCH(EPL)                                                                                  \
    hipLaunchKernelGGL((topk_windows_kernel<EPL, false>), grid, block, 0, s, scores, scores_layer_stride, seg_off, \
                       seg_len, topk_len, n_req, start_w, end_w, idx_out, out_stride, count_out, block_tables, \
                       bt_stride, phys_out, seq_lens, block_size, sparse_seq_lens)
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
    UCM_LAUNCH_CHECK("ucm_topk_windows");
}

extern "C" int ucm_kvstar_topk(const float* votes, const int32_t* seg_off, const int32_t* seg_len,
                               const int32_t* topk_len, int n_tasks, int max_seg_len, int32_t* idx_out,
                               int out_stride, int32_t* count_out, ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks >= 0 && max_seg_len >= 0, "ucm_kvstar_topk: n_tasks=%d max_seg_len=%d", n_tasks, max_seg_len);
    if (n_tasks == 0) { return UCM_OK; }
    UCM_REQUIRE(votes && seg_off && seg_len && topk_len && idx_out && count_out, "ucm_kvstar_topk: null pointer");
    UCM_REQUIRE(out_stride >= max_seg_len, "ucm_kvstar_topk: out_stride=%d < max_seg_len=%d", out_stride, max_seg_len);
    UCM_SUPPORTED(max_seg_len <= 4096, "ucm_kvstar_topk: max_seg_len=%d (at most 4096 blocks per task)", max_seg_len);
    hipStream_t s = ucm::as_stream(stream);
    const dim3 grid(n_tasks, 1), block(64);
#define UCM_HEAP_LAUNCH(EPL)                                                                                   \
    hipLaunchKernelGGL((topk_windows_kernel<EPL, true>), grid, block, 0, s, votes, int64_t{0}, seg_off, seg_len, \
                       topk_len, n_tasks, 0, 0, idx_out, out_stride, count_out, nullptr, 0, nullptr, nullptr, 1, \
                       nullptr)
    if (max_seg_len <= 64) { UCM_HEAP_LAUNCH(1); }
    else if (max_seg_len <= 128) { UCM_HEAP_LAUNCH(2); }
    else if (max_seg_len <= 256) { UCM_HEAP_LAUNCH(4); }
    else if (max_seg_len <= 512) { UCM_HEAP_LAUNCH(8); }
    else if (max_seg_len <= 1024) { UCM_HEAP_LAUNCH(16); }
    else if (max_seg_len <= 2048) { UCM_HEAP_LAUNCH(32); }
    else { UCM_HEAP_LAUNCH(64); }
#undef UCM_HEAP_LAUNCH
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
    const float* __restrict__ votes, const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len,
    int32_t* __restrict__ idx, int out_stride, const int32_t* __restrict__ count)
{
    __shared__ unsigned long long keys[kOrderMax];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int k = min(count[t], min(out_stride, kOrderMax));
    const int n = seg_len[t];
    int32_t* row = idx + static_cast<size_t>(t) * out_stride;
    const float* v = votes + seg_off[t];
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

extern "C" int ucm_kvstar_order(const float* votes, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                                int max_count, int32_t* idx_io, int out_stride, const int32_t* count,
                                ucm_stream_t stream)
{
    UCM_REQUIRE(n_tasks >= 0 && max_count >= 0, "ucm_kvstar_order: n_tasks=%d max_count=%d", n_tasks, max_count);
    if (n_tasks == 0 || max_count == 0) { return UCM_OK; }
    UCM_REQUIRE(votes && seg_off && seg_len && idx_io && count, "ucm_kvstar_order: null pointer");
    UCM_REQUIRE(out_stride >= max_count, "ucm_kvstar_order: out_stride=%d < max_count=%d", out_stride, max_count);
    UCM_SUPPORTED(max_count <= kOrderMax, "ucm_kvstar_order: max_count=%d (at most 4096 chosen blocks per task)", max_count);
    hipLaunchKernelGGL(kvstar_order_kernel, dim3(n_tasks), dim3(kOrderThreads), 0, ucm::as_stream(stream), votes, seg_off,
                       seg_len, idx_io, out_stride, count);
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
