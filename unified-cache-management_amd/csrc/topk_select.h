// Block selection of one (layer, request) by one 64-wide wavefront: the device
// function behind ucm_topk_windows / ucm_kvstar_topk (topk.hip) and behind the
// tail of the fused score + select kernel (score.hip).
//
// The request's scores are held in registers as order-preserving 32-bit keys
// (element i lives in lane i%64, register i/64).  Selection is a radix select,
// one bit per step from the top: the threshold T is grown greedily while at
// least m candidates have key >= T, each count being a wave ballot + popcount.
// Candidates with key > T are all taken; of those with key == T the first
// `m - count(key > T)` in index order are taken, which is exactly where a
// stable descending sort leaves equal scores.  Output positions are ballot
// prefix counts in index order, so the result comes out sorted ascending with
// no sort at all, and the logical->physical block-table lookup is applied on
// the way out.
#pragma once

#include "common.h"

namespace ucm {

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

// What one selection reads and writes; the same for every (layer, request) of a launch.
struct SelectArgs {
    const float* scores;            // layer 0; row x of layer l at scores[l * scores_layer_stride + x]
    int64_t scores_layer_stride;
    int64_t scores_rows;            // rows of a layer that may be read: a request outside them selects nothing
    const int32_t* seg_off;
    const int32_t* seg_len;
    const int32_t* topk_len;
    int n_req;
    int max_seg_len;                // the host's bound: a longer seg_len is cut there
    int start_w, end_w;
    int32_t* idx_out;
    int out_stride;
    int64_t idx_layer_stride;       // elements between two layers of idx_out / phys_out (dense: n_req * out_stride)
    int64_t cnt_layer_stride;       // elements between two layers of count_out / sparse_seq_lens (dense: n_req)
    int32_t* count_out;
    const int32_t* block_tables;
    int bt_stride;
    int32_t* phys_out;
    const int32_t* seq_lens;
    int block_size;
    int32_t* sparse_seq_lens;
};

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
// Called by all 64 lanes of one wave for request r of layer l; kEpl * 64 is the
// longest request the instance holds (longer ones are cut there: host checked).
//
// kCoherent: the scores were written by other workgroups of the SAME launch (device-scope stores that went through
// to memory); they are read with device-scope loads, which do not take a line that an L2 of another part of the
// chip may still hold in an older state.
template <int kEpl, bool kHeapTies, bool kCoherent = false>
__device__ __forceinline__ void select_wave(const SelectArgs& a, int r, int l, int lane)
{
    const int start_w = a.start_w, end_w = a.end_w, out_stride = a.out_stride;
    const int64_t lr = static_cast<int64_t>(l) * a.cnt_layer_stride + r;
    const int64_t row_at = static_cast<int64_t>(l) * a.idx_layer_stride + static_cast<int64_t>(r) * out_stride;
    int n = a.seg_len[r];
    n = min(min(n, a.max_seg_len), min(out_stride, 64 * kEpl));  // host checked; clamp so nothing can run past a row
    if (a.block_tables) { n = min(n, a.bt_stride); }
    const int64_t seg0 = a.seg_off[r];
    // a descriptor that came from device memory is followed only inside the scores of a layer
    if (seg0 < 0 || seg0 + max(n, 0) > a.scores_rows) { n = 0; }
    const int k = a.topk_len[r];
    int32_t* out = a.idx_out + row_at;
    int32_t* pout = a.phys_out ? a.phys_out + row_at : nullptr;
    const int32_t* bt = a.block_tables ? a.block_tables + static_cast<size_t>(r) * a.bt_stride : nullptr;
    int count = 0;
    bool kept_all = false;

    if (n <= 0) {
        count = 0;
        kept_all = true;                         // nothing to drop: the request keeps its length
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
        const float* s = a.scores + static_cast<int64_t>(l) * a.scores_layer_stride + seg0;
        unsigned key[kEpl];
        int32_t phys[kEpl];                      // the block table's entries, fetched with the scores: a load per
#pragma unroll                                   // taken element on the way out would cost a memory round trip per register
        for (int j = 0; j < kEpl; ++j) {
            const int i = j * 64 + lane;
            const bool cand = i >= start_w && i < hi;
            const float* sp = s + (cand ? i : 0);
            const float sv = kCoherent ? __hip_atomic_load(sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *sp;
            key[j] = cand ? ordered_key(sv) : 0u;
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
        a.count_out[lr] = count;
        if (a.sparse_seq_lens && a.seq_lens) {
            const int len = a.seq_lens[r], rem = len % a.block_size;
            // every block kept: the request keeps its length; otherwise `count` blocks, the last one partial
            a.sparse_seq_lens[lr] = kept_all ? len : (rem == 0 ? count * a.block_size : count * a.block_size - a.block_size + rem);
        }
    }
}

}  // namespace ucm
