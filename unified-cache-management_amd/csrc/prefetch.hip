// Hit / miss / free-list bookkeeping of the GSA prefetch engine on the device:
// GSAPrefetchEngineC::RunOneBsPrefetch with GetHitAndMissBlock, RunPrefetchH2D
// and LoadKVToHBM (ucm/sparse/gsa/prefetch/src/kvcache_pre.cpp:206-322), one
// 256-thread workgroup per (request of the call, layer).
//
// The reference walks std::map / std::unordered_set containers with 16 OpenMP
// threads over the layers, requests one after the other.  Here a request's
// resident blocks are a row of plain arrays (slot s: cache block map_block[s],
// logical block map_idx[l][s]) and every step of the walk is a rank:
//   * a selected logical block is a hit if some slot holds it (each thread
//     scans the slots for one selection entry); misses keep their top-k order
//     (rank = misses before it, a ballot prefix);
//   * a free-list entry is eligible if its block is not (yet) in the hit set;
//     the i-th eligible entry, in free-list order, takes the i-th miss;
//   * the success table lists hits and served misses by logical index
//     ascending (rank = entries with a smaller index);
//   * the new free list is the blocks outside the hit set by block id ascending
//     (rank = such blocks with a smaller id).
// A few hundred integers per workgroup: latency-bound, like the selection.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

__device__ __forceinline__ unsigned lanes_below(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u));
}

// Rank of this thread among the threads (in thread order) whose predicate holds, and their number.
__device__ __forceinline__ int block_rank(bool pred, int* s_cnt, int& total)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned long long mask = __ballot(pred);
    int rank = static_cast<int>(lanes_below(mask));
    __syncthreads();                                   // s_cnt may still be read from the previous use
    if (lane == 0) { s_cnt[wave] = __popcll(mask); }
    __syncthreads();
    total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        if (w < wave) { rank += s_cnt[w]; }
        total += s_cnt[w];
    }
    return rank;
}

// grid: x = request of the call, y = layer
__global__ __launch_bounds__(kThreads) void prefetch_plan_kernel(
    const int32_t* __restrict__ map_block, const int32_t* __restrict__ map_len, int32_t* __restrict__ map_idx,
    int table_rows, int cap, const int32_t* __restrict__ topk_idx, int topk_stride,
    const int32_t* __restrict__ topk_len, const int32_t* __restrict__ rows, const int32_t* __restrict__ bs_index,
    int batch, int max_bs, int row_len, int32_t* __restrict__ free_block, int32_t* __restrict__ free_len,
    int32_t* __restrict__ success_blocks, int32_t* __restrict__ success_len, int32_t* __restrict__ load_blocks,
    int32_t* __restrict__ load_count, int32_t* __restrict__ miss_idxs, int32_t* __restrict__ miss_count)
{
    __shared__ int32_t s_block[kThreads], s_idx[kThreads], s_miss[kThreads];
    __shared__ int32_t s_ent_idx[2 * kThreads], s_ent_blk[2 * kThreads], s_succ[2 * kThreads];
    __shared__ int s_hit[kThreads];
    __shared__ int s_cnt[kWaves];

    const int i = blockIdx.x, l = blockIdx.y, t = threadIdx.x;
    const size_t li = static_cast<size_t>(l) * batch + i;
    const int row = rows[i], b = bs_index[i];
    const int k = min(min(topk_len[i], topk_stride), kThreads);
    if (row < 0 || row >= table_rows || b < 0 || b >= max_bs || k <= 0) {   // (uniform) the reference skips such a request
        if (t == 0 && row >= 0 && row < table_rows) {
            load_count[static_cast<size_t>(l) * table_rows + row] = 0;
            miss_count[static_cast<size_t>(l) * table_rows + row] = 0;
        }
        return;
    }
    const size_t lb = static_cast<size_t>(l) * max_bs + b;
    const size_t lr = static_cast<size_t>(l) * table_rows + row;     // results stay with the request's row
    const int n = min(min(map_len[row], cap), kThreads);
    const int f = min(min(free_len[lb], row_len), kThreads);
    int32_t* idx_row = map_idx + (static_cast<size_t>(l) * table_rows + row) * cap;
    int32_t* free_row = free_block + lb * row_len;
    int32_t* succ_row = success_blocks + lb * row_len;

    s_block[t] = t < n ? map_block[static_cast<size_t>(row) * cap + t] : -1;
    s_idx[t] = t < n ? idx_row[t] : -1;
    s_hit[t] = 0;
    const int item = t < k ? topk_idx[li * topk_stride + t] : -1;
    const int free_id = t < f ? free_row[t] : -1;
    s_succ[t] = 0;
    s_succ[t + kThreads] = 0;
    __syncthreads();

    // 1. hits and misses of the selection
    int hit_slot = -1;
    if (t < k) {
        for (int s = 0; s < n; ++s) {
            if (s_idx[s] == item) { hit_slot = s; break; }
        }
        if (hit_slot >= 0) { s_hit[hit_slot] = 1; }
    }
    const bool is_hit = t < k && hit_slot >= 0, is_miss = t < k && hit_slot < 0;
    int n_hit_entries, n_miss;
    const int hit_rank = block_rank(is_hit, s_cnt, n_hit_entries);
    const int miss_rank = block_rank(is_miss, s_cnt, n_miss);
    if (is_miss) {
        s_miss[miss_rank] = item;
        miss_idxs[lr * topk_stride + miss_rank] = item;
    }
    if (is_hit) { s_ent_idx[hit_rank] = item; s_ent_blk[hit_rank] = s_block[hit_slot]; }
    __syncthreads();                                   // s_hit, s_miss complete

    // 2. the free list serves the misses in order
    int free_slot = -1;
    if (t < f) {
        for (int s = 0; s < n; ++s) {
            if (s_block[s] == free_id) { free_slot = s; break; }
        }
    }
    const bool eligible = n_miss > 0 && free_slot >= 0 && s_hit[free_slot] == 0;
    int n_eligible;
    const int el_rank = block_rank(eligible, s_cnt, n_eligible);
    const int n_load = min(min(n_eligible, n_miss), cap);   // (a free list that names a block twice could outnumber the slots)
    if (eligible && el_rank < n_load) {
        const int32_t want = s_miss[el_rank];
        load_blocks[lr * cap + el_rank] = free_id;
        s_hit[free_slot] = 1;
        s_idx[free_slot] = want;                          // the block now holds the missing logical block
        s_ent_idx[n_hit_entries + el_rank] = want;
        s_ent_blk[n_hit_entries + el_rank] = free_id;
    }
    __syncthreads();

    // 3. success table: by logical index ascending
    const int n_ent = n_hit_entries + n_load;
    for (int e = t; e < n_ent; e += kThreads) {
        const int32_t mine = s_ent_idx[e];
        int rank = 0;
        for (int u = 0; u < n_ent; ++u) { rank += s_ent_idx[u] < mine ? 1 : 0; }
        s_succ[rank] = s_ent_blk[e];
    }
    __syncthreads();
    // (the reference zero-fills the whole row first)
    for (int p = t; p < row_len; p += kThreads) { succ_row[p] = p < 2 * kThreads ? s_succ[p] : 0; }

    // 4. new free list: blocks outside the hit set by block id ascending; map write-back
    const bool is_free = t < n && s_hit[t] == 0;
    if (is_free) {
        const int32_t mine = s_block[t];
        int rank = 0;
        for (int u = 0; u < n; ++u) { rank += (s_hit[u] == 0 && s_block[u] < mine) ? 1 : 0; }
        if (rank < row_len) { free_row[rank] = mine; }
    }
    int n_free, n_in_hit;
    block_rank(is_free, s_cnt, n_free);
    block_rank(t < n && s_hit[t] != 0, s_cnt, n_in_hit);
    if (t < n) { idx_row[t] = s_idx[t]; }
    if (t == 0) {
        free_len[lb] = n_free;
        success_len[lb] = n_in_hit;
        load_count[lr] = n_load;
        miss_count[lr] = n_miss;
    }
}

}  // namespace

extern "C" int ucm_prefetch_plan(const int32_t* map_block, const int32_t* map_len, int32_t* map_idx, int table_rows,
                                 int cap, const int32_t* topk_idx, int topk_stride, const int32_t* topk_len,
                                 const int32_t* rows, const int32_t* bs_index, int batch, int n_layers, int max_bs,
                                 int row_len, int32_t* free_block, int32_t* free_len, int32_t* success_blocks,
                                 int32_t* success_len, int32_t* load_blocks, int32_t* load_count, int32_t* miss_idxs,
                                 int32_t* miss_count, ucm_stream_t stream)
{
    UCM_REQUIRE(batch >= 0 && n_layers > 0 && n_layers <= 65535, "ucm_prefetch_plan: batch=%d n_layers=%d", batch, n_layers);
    if (batch == 0) { return UCM_OK; }
    UCM_REQUIRE(map_block && map_len && map_idx && topk_idx && topk_len && rows && bs_index && free_block && free_len &&
                    success_blocks && success_len && load_blocks && load_count && miss_idxs && miss_count,
                "ucm_prefetch_plan: null pointer");
    UCM_REQUIRE(table_rows > 0 && max_bs > 0, "ucm_prefetch_plan: table_rows=%d max_bs=%d", table_rows, max_bs);
    UCM_SUPPORTED(cap >= 1 && cap <= kThreads && topk_stride >= 1 && topk_stride <= kThreads && row_len >= 1,
                  "ucm_prefetch_plan: cap=%d topk_stride=%d (1..%d resident blocks and selected blocks per request)", cap,
                  topk_stride, kThreads);
    hipLaunchKernelGGL(prefetch_plan_kernel, dim3(batch, n_layers), dim3(kThreads), 0, ucm::as_stream(stream), map_block,
                       map_len, map_idx, table_rows, cap, topk_idx, topk_stride, topk_len, rows, bs_index, batch, max_bs,
                       row_len, free_block, free_len, success_blocks, success_len, load_blocks, load_count, miss_idxs,
                       miss_count);
    UCM_LAUNCH_CHECK("ucm_prefetch_plan");
}
