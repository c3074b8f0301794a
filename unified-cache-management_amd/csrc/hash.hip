// Hash-code retrieval (KvComp style): sign-random-projection codes of the keys,
// per-block summaries of those codes, query codes, and integer block scores.
//
// The projection [vectors x 128] . [128 x 128] is the one real contraction on
// the whole retrieval path (128 flop per byte of key), so it runs on the matrix
// cores: v_mfma_f32_32x32x16_bf16, one wave per cache block, 32-vector tiles,
// the weight matrix staged once per workgroup in LDS (transposed, padded rows,
// sign flipped).
// Only the SIGN of each projection is kept, and it has to be the sign of the
// exactly accumulated dot product (the CPU oracle accumulates in fp64), so
// every result whose magnitude is within the fp32 accumulation error bound
//     |acc| < 2^-16 * ||x|| * ||w_c||
// is queued and redone by one lane in fp64, d ascending; one or two bits per
// ten thousand take that path (the bound uses the largest column norm of each
// 32-column block; a min over a lane's sixteen results flags blocks, and only
// flagged ones get the per-result look).  The bound holds for any order of
// the 127 additions with each one off by up to a whole unit in the last place
// (truncation): 127 * 2^-23 * sum|x_d w_d| < 2^-16 * ||x|| ||w_c||, the
// products of two bf16 values being exact in fp32.  (Measured on gfx950 with
// the redo switched off: no sign of 1.5e9 Gaussian, wide-range or pairwise
// cancelling projections differs from the exact one above 2^-26 ||x|| ||w_c||.)
// The next tile's keys are in flight while the current one goes through the
// matrix cores.
//
// Per cache block the kernel emits: the token codes (LSB-first packing: bit j
// of byte b is column 8b+j), the per-(kv head, bit) column sums over the
// block's tokens S[h][c] = #ones - #zeros, and the majority-vote block code
// (bit c of head h = S[h][c] > 0).  Both block scores used downstream are
// integer functions of these: the reference's sum over all (query head, kv
// head, token) of +-1 inner products equals <sum_i u(q_i), sum_h S[h]>.
#include <algorithm>

#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kDim = 128;           // head_dim
constexpr int kBits = 128;          // code length
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kWtStride = kDim + 8; // bf16 elements per transposed weight row (272 B: spreads LDS banks)
constexpr int kQueueCap = 256;
constexpr int kMaxHeads = 8;
constexpr float kTau2 = 0x1p-30f;   // (2^-15)^2: the query kernel's bound (three bf16 terms per mean, added afterwards)
constexpr float kTauBlocks2 = 0x1p-32f;   // (2^-16)^2: the block kernel's bound (one chain of 127 additions per result)

__device__ __forceinline__ unsigned lanes_below(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u));
}

// row of the staged (negated, transposed) weight matrix that holds weight column `col`:
// within its 32-column block, column half*16 + i sits in row (i/4)*8 + half*4 + i%4
__device__ __forceinline__ int row_of_col(int col)
{
    const int cb = col & 31, h = cb >> 4, i = cb & 15;
    return (col & ~31) + (i >> 2) * 8 + h * 4 + (i & 3);
}

struct __attribute__((aligned(16))) WaveScratch {
    unsigned queue[kQueueCap];
    int colsum[kMaxHeads][kBits];   // per-head ones counts of the block being encoded
};

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// Keys, queries and weights are bfloat16 (kF16 false) or float16 (true): a model's own type.  What the two share:
// 16-bit elements with the sign in bit 15, products of two of them exact in fp32 (8 x 8 or 11 x 11 significant
// bits; the smallest float16 product, 2^-48, is a normal fp32 number, and the matrix instruction takes float16
// subnormals as they are), a matrix instruction of the same shape.
template <bool kF16>
__device__ __forceinline__ float dot2_self(unsigned e, float s)
{
    if (kF16) { const f16x2 p = __builtin_bit_cast(f16x2, e); return __builtin_amdgcn_fdot2(p, p, s, false); }
    const bf16x2 p = __builtin_bit_cast(bf16x2, e);
    return __builtin_amdgcn_fdot2_f32_bf16(p, p, s, false);
}

// the two 16-bit elements of a word, widened exactly
template <bool kF16>
__device__ __forceinline__ float widen_lo(unsigned e)
{
    if (kF16) { return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(e & 0xffffu))); }
    return __uint_as_float(e << 16);
}
template <bool kF16>
__device__ __forceinline__ float widen_hi(unsigned e)
{
    if (kF16) { return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(e >> 16))); }
    return __uint_as_float(e & 0xffff0000u);
}

template <bool kF16>
__device__ __forceinline__ f32x16 mfma_32x32x16(const u32x4 a, const u32x4 b, const f32x16 c)
{
    if (kF16) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0); }
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// sum of squares of 8 elements added to s (v_dot2c_f32_bf16 / v_dot2_f32_f16); only used for error bounds
template <bool kF16>
__device__ __forceinline__ float norm2_acc(const u32x4 v, float s)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned e = v[j];   // (a bit_cast of v[j] itself reads element 0 four times with this compiler)
        s = dot2_self<kF16>(e, s);
    }
    return s;
}

// Exact sign of x . W[:, col] from the NEGATED weight row kept in LDS: fp64
// accumulation, d ascending (the oracle's order; negation is exact and
// rounding is symmetric, so the sum is the oracle's with its sign flipped).
// Both 256-byte rows are fetched with sixteen 16-byte loads issued together, so
// the redo costs one memory latency, not 128 of them.
template <bool kF16>
__device__ __forceinline__ bool exact_positive(const unsigned short* __restrict__ x,
                                               const unsigned short* __restrict__ neg_wt_col)
{
    u32x4 xv[kDim / 8], wv[kDim / 8];
#pragma unroll
    for (int i = 0; i < kDim / 8; ++i) {
        xv[i] = ucm::gload16(x + i * 8);
        wv[i] = *reinterpret_cast<const u32x4*>(neg_wt_col + i * 8);
    }
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < kDim / 8; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned xa = xv[i][j], wa = wv[i][j];
            // (a product of two such values is exact in fp64, so the fused form rounds exactly as multiply-then-add does)
            acc = __builtin_fma(static_cast<double>(widen_lo<kF16>(xa)), static_cast<double>(widen_lo<kF16>(wa)), acc);
            acc = __builtin_fma(static_cast<double>(widen_hi<kF16>(xa)), static_cast<double>(widen_hi<kF16>(wa)), acc);
        }
    }
    return acc < 0.0;
}

// Queued results are redone exactly, 64 at a time, one per lane.  Entries are
// queued after their tile's code words were stored, so the fix goes to memory.
// Kept out of line: it has several call sites and runs rarely.
template <bool kF16>
__device__ __attribute__((noinline)) void drain_exact(WaveScratch& ws, int qlen, int lane,
                                                      const unsigned short* __restrict__ blk,
                                                      const unsigned short* __restrict__ neg_wt,
                                                      unsigned* __restrict__ tc_out, unsigned kv_heads)
{
    // the code words stored by this wave must have reached L2 before they are patched there;
    // waiting for the stores' acknowledgements is enough (a device-scope fence would write back the whole L2)
    if (tc_out) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
    }
    for (int base = 0; base < qlen; base += 64) {
        if (base + lane < qlen) {
            const unsigned e = ws.queue[base + lane];
            const unsigned v = e >> 8, col = (e >> 1) & 127u, prov = e & 1u;
            const bool pos = exact_positive<kF16>(blk + static_cast<size_t>(v) * kDim, &neg_wt[row_of_col(col) * kWtStride]);
            if (static_cast<unsigned>(pos) != prov) {
                if (tc_out) { atomicXor(&tc_out[v * 4 + (col >> 5)], 1u << (col & 31)); }
                atomicAdd(&ws.colsum[v % kv_heads][col], pos ? 1 : -1);
            }
        }
    }
}

// Bit-sliced counters: plane p holds bit p of 32 independent counts, one per bit
// position of the words added.  Six planes count to 63.
constexpr int kPlanes = 6;
constexpr unsigned kFlushTiles = 63;

__device__ __forceinline__ void planes_add(unsigned (&pl)[kPlanes], unsigned x)
{
#pragma unroll
    for (int p = 0; p < kPlanes; ++p) {
        const unsigned carry = pl[p] & x;
        pl[p] ^= x;
        x = carry;
    }
}

// Adds the 32 counts of a plane set to the per-head column sums in LDS and clears
// it.  Bit b of word pair `wp` is column (2*wp + b/16)*32 + half*16 + b%16.
__device__ __forceinline__ void planes_flush(unsigned (&pl)[kPlanes], int* __restrict__ head_row, int wp, int half)
{
#pragma unroll 4
    for (int b = 0; b < 32; ++b) {
        int cnt = 0;
#pragma unroll
        for (int p = 0; p < kPlanes; ++p) { cnt |= static_cast<int>((pl[p] >> b) & 1u) << p; }
        const int col = (2 * wp + (b >> 4)) * 32 + half * 16 + (b & 15);
        if (cnt) { atomicAdd(&head_row[col], cnt); }
    }
#pragma unroll
    for (int p = 0; p < kPlanes; ++p) { pl[p] = 0u; }
}

// The same without atomics, for kHeads = 8, 4, 2 or 1 kv heads: the 32 / kHeads lanes of a lane half that hold
// vectors of one head (lr, lr ^ kHeads, lr ^ 2 kHeads, ...) first add their counts up across lanes - as bytes, four
// to a register, for the first two levels (a plane set counts at most 63 tiles, four lanes 252), as halfwords for the
// levels beyond - and lane lr < kHeads then owns head lr's sixteen columns of each of the two column blocks outright.
// (Thirty-two LDS atomics per lane, with 32 / kHeads lanes on every address, took four times as long as everything
// else a block of eight heads needs at its end, and more than the block's tiles for one head.)
// x + (x of the lane kS away), for sums over the lanes lr, lr +- kS, lr +- 2 kS, ... of a 32-lane half: within a row
// of sixteen lanes a rotation by kS (a DPP operand, no LDS), and for kS = 16 the row exchange of v_permlane16_swap
// (rows 1 and 3 of one copy against rows 0 and 2 of another, so the two results add up to the pair's sum in both).
template <int kS>
__device__ __forceinline__ unsigned coset_add(unsigned x)
{
    if constexpr (kS == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
        return r[0] + r[1];
    } else {
        return x + static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x120 + kS, 0xf, 0xf, false));
    }
}

template <int kHeads>
__device__ __forceinline__ void planes_flush_owner(unsigned (&pl)[kPlanes], int* __restrict__ colsum, int wp, int half, int lr)
{
    typedef int i32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int j = 0; j < 8; ++j) {                        // bits 4j .. 4j+3: columns (2*wp + j/4)*32 + half*16 + 4*(j%4) + 0..3
        unsigned c = 0u;                                 // byte k: count of bit 4j + k
#pragma unroll
        for (int p = 0; p < kPlanes; ++p) {
            const unsigned nib = (pl[p] >> (4 * j)) & 0xfu;
            c += ((nib * 0x00204081u) & 0x01010101u) << p;   // bit i of the nibble -> byte i
        }
        c = coset_add<kHeads>(c);
        c = coset_add<2 * kHeads>(c);
        unsigned even = c & 0x00ff00ffu, odd = (c >> 8) & 0x00ff00ffu;   // counts of bits 4j, 4j+2 / 4j+1, 4j+3
        if constexpr (kHeads <= 1) { even = coset_add<4>(even); odd = coset_add<4>(odd); }
        if constexpr (kHeads <= 2) { even = coset_add<8>(even); odd = coset_add<8>(odd); }
        if constexpr (kHeads <= 4) { even = coset_add<16>(even); odd = coset_add<16>(odd); }
        if (lr < kHeads) {
            int* dst = colsum + lr * kBits + (2 * wp + (j >> 2)) * 32 + half * 16 + 4 * (j & 3);
            i32x4 v = *reinterpret_cast<i32x4*>(dst);
            v.x += static_cast<int>(even & 0xffffu);
            v.y += static_cast<int>(odd & 0xffffu);
            v.z += static_cast<int>(even >> 16);
            v.w += static_cast<int>(odd >> 16);
            *reinterpret_cast<i32x4*>(dst) = v;
        }
    }
#pragma unroll
    for (int p = 0; p < kPlanes; ++p) { pl[p] = 0u; }
}

// The product is taken transposed, C^T = (-W)^T . X^T: the matrix cores' A
// operand is the (negated) weight fragment and B the key fragment, so that lane
// (half, lr) ends up with sixteen results per 32-column block of ITS OWN vector
// lr in registers: accumulator i of block nb is row (i/4)*8 + half*4 + i%4 of
// the block's A operand.  Which weight column a row of A holds is free: the
// staged copy keeps column nb*32 + half*16 + i in that row (row_of_col below),
// so a lane's sixteen results are sixteen ADJACENT columns and the code words
// need no bit shuffling: accumulator i of block nb is column
//     nb*32 + half*16 + i.
// With the weights negated, a projection is positive exactly when its
// accumulator has the sign bit set (and an all-zero key gives +0: bit clear), so
// one v_alignbit per result shifts the bit into the lane's code word, the two
// halves are merged with one cross-lane move, and the per-column counts over a
// block's tokens are kept in bit-sliced counters (a lane's vectors all belong to
// one kv head because kv_heads divides 32) that are added to LDS once per block.
// Workgroups are persistent over the list of blocks so that staging the weight
// matrix is paid once per workgroup, not once per four blocks.
// grid: x = workgroup (wave w of workgroup g takes items g*kWaves + w, then steps by the grid), y = layer
template <bool kTokenCodes, bool kF16>
__global__ __launch_bounds__(kThreads, 2) void hash_encode_blocks_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned n_items, unsigned rows,
    unsigned tokens, unsigned kv_heads, const unsigned short* __restrict__ w,
    unsigned* __restrict__ token_codes, int64_t tc_layer_stride,
    short* __restrict__ colsum_out, int64_t cs_layer_stride,
    unsigned* __restrict__ block_codes, int64_t bc_layer_stride)
{
    __shared__ __attribute__((aligned(16))) unsigned short wt[kBits * kWtStride];  // wt[row_of_col(col)][d] = -W[d][col]
    __shared__ float w_norm2[kBits];                     // by row of wt
    __shared__ WaveScratch scratch[kWaves];

    // ---- weights: global [d][col] -> LDS [col][d], sign flipped
    for (int e8 = threadIdx.x; e8 < kDim * kBits / 8; e8 += kThreads) {
        const int d = e8 / (kBits / 8), c0 = (e8 % (kBits / 8)) * 8;
        const u32x4 v = *reinterpret_cast<const u32x4*>(w + d * kBits + c0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            wt[row_of_col(c0 + 2 * j) * kWtStride + d] = static_cast<unsigned short>((v[j] & 0xffffu) ^ 0x8000u);
            wt[row_of_col(c0 + 2 * j + 1) * kWtStride + d] = static_cast<unsigned short>((v[j] >> 16) ^ 0x8000u);
        }
    }
    __syncthreads();
    {
        const int c = threadIdx.x >> 1, part = threadIdx.x & 1;   // two threads per column, 64 dims each
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            s = norm2_acc<kF16>(*reinterpret_cast<const u32x4*>(&wt[c * kWtStride + part * 64 + k * 8]), s);
        }
        s += __shfl_xor(s, 1, 64);
        if (part == 0) { w_norm2[c] = s; }
    }
    __syncthreads();

    // the wave index through readfirstlane: the item a wave works on is then known to be the same for all lanes,
    // and its block id and slot are read with scalar loads, which do not queue behind the key loads in flight
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int half = lane >> 5, lr = lane & 31;
    const unsigned l = blockIdx.y;
    const unsigned n_vec = tokens * kv_heads;            // vectors of kDim bf16 in a block
    const unsigned n_tiles = n_vec / 32;
    WaveScratch& ws = scratch[wave];
    int* head_row = &ws.colsum[lr % kv_heads][0];        // vector tile*32 + lr is a row of head lr % kv_heads

    float sw[4];                                         // tau * largest ||w_col|| of each 32-column block
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
        float m = w_norm2[nb * 32 + lr];
#pragma unroll
        for (int d = 16; d >= 1; d >>= 1) { m = fmaxf(m, __shfl_xor(m, d, 64)); }
        sw[nb] = sqrtf(kTauBlocks2 * m) * 1.0001f;
    }

    // keys of item i, or null when its block id or slot is out of range (never dereferenced)
    auto item_keys = [&](unsigned i, unsigned& slot_out) -> const unsigned short* {
        if (i >= n_items) { return nullptr; }
        const unsigned id = block_ids ? static_cast<unsigned>(block_ids[i]) : i;
        slot_out = slots ? static_cast<unsigned>(slots[i]) : i;
        if (id >= num_blocks || slot_out >= rows) { return nullptr; }
        return static_cast<const unsigned short*>(k_layers[l]) + static_cast<size_t>(id) * n_vec * kDim;
    };

    // B fragments (keys).  MFMA step ks of lane (vector lr, k-half `half`) takes dims
    // ks*16 + half*8 .. +8, the instruction's own order: the two lanes of a vector then
    // read neighbouring 16-byte pieces of one 32-byte sector in every load instruction, so
    // an instruction touches 32 cache lines, not 64.  (With a lane reading its own
    // contiguous 128-byte line over the eight steps instead - half*64 + ks*8, any order
    // of the contraction index being fine as long as both operands agree - the kernel
    // took 12 % more cycles with the keys from HBM and the same with the keys in cache.)
    u32x4 k_a[8], k_b[8];
    auto load_tile = [&](u32x4 (&kf)[8], const unsigned short* from, unsigned tile) {
        const unsigned short* xrow = from + (static_cast<size_t>(tile) * 32 + lr) * kDim + half * 8;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) { kf[ks] = ucm::gload16(xrow + ks * 16); }
    };
    bool prefetched = false;                             // k_a / k_b already hold (or await) this item's first tiles

    const unsigned item_step = gridDim.x * kWaves;
    const unsigned first_item = blockIdx.x * kWaves + wave;
    unsigned carried_slot = 0;                           // the item looked up as the one before's successor
    const unsigned short* carried_blk = item_keys(first_item, carried_slot);
    for (unsigned item = first_item; item < n_items; item += item_step) {
        unsigned next_slot = 0;
        const unsigned slot = carried_slot;
        const unsigned short* blk = carried_blk;
        // the tiles after this item's last one come from the next item of this wave, so its
        // first keys are on their way while this item's summaries are written
        const unsigned short* next_blk = item_keys(item + item_step, next_slot);
        carried_blk = next_blk;
        carried_slot = next_slot;
        if (!blk) { prefetched = false; continue; }
        const bool chain = next_blk != nullptr && n_tiles >= 2;
        if (!chain) { next_blk = blk; }
        unsigned* tc_out = kTokenCodes ? token_codes + (static_cast<int64_t>(l) * tc_layer_stride +
                                                        static_cast<int64_t>(slot) * n_vec * 4) : nullptr;
        for (int e = lane; e < kMaxHeads * kBits; e += 64) { (&ws.colsum[0][0])[e] = 0; }

        unsigned planes01[kPlanes], planes23[kPlanes];
#pragma unroll
        for (int p = 0; p < kPlanes; ++p) { planes01[p] = 0u; planes23[p] = 0u; }
        unsigned pending = 0;                            // tiles counted in the planes
        int qlen = 0;
        // inside a block of more than 63 tiles (once per 63 tiles; the three copies of the tile code each hold one)
        auto flush_planes = [&]() {
            if (kv_heads == 8) {                         // (uniform)
                planes_flush_owner<8>(planes01, &ws.colsum[0][0], 0, half, lr);
                planes_flush_owner<8>(planes23, &ws.colsum[0][0], 1, half, lr);
            } else {
                planes_flush(planes01, head_row, 0, half);
                planes_flush(planes23, head_row, 1, half);
            }
        };
        // at the end of every block
        auto flush_planes_last = [&]() {
            switch (kv_heads) {                          // (uniform)
            case 8: planes_flush_owner<8>(planes01, &ws.colsum[0][0], 0, half, lr); planes_flush_owner<8>(planes23, &ws.colsum[0][0], 1, half, lr); break;
            case 4: planes_flush_owner<4>(planes01, &ws.colsum[0][0], 0, half, lr); planes_flush_owner<4>(planes23, &ws.colsum[0][0], 1, half, lr); break;
            case 2: planes_flush_owner<2>(planes01, &ws.colsum[0][0], 0, half, lr); planes_flush_owner<2>(planes23, &ws.colsum[0][0], 1, half, lr); break;
            default: planes_flush_owner<1>(planes01, &ws.colsum[0][0], 0, half, lr); planes_flush_owner<1>(planes23, &ws.colsum[0][0], 1, half, lr); break;
            }
        };

        // A tile's code words are stored one trip late, at the start of the next tile's work:
        // a store issued just before the wait for the next keys would be waited for as well.
        // The store is unconditional (a branch around it would make the compiler's wait-count
        // bookkeeping pessimistic): the first trip writes zeros to tile 0's slot, which the
        // second trip overwrites.  The exact redo patches code words in memory, so what is
        // held here is stored before a drain and read back after it.
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        u32x2 pend_cw = {0u, 0u};
        unsigned pend_tile = 0;
        auto store_codes = [&]() {
            if (kTokenCodes) {
                *reinterpret_cast<u32x2*>(tc_out + (static_cast<size_t>(pend_tile) * 32 + lr) * 4 + half * 2) = pend_cw;
            }
        };
        auto drain_queue = [&]() {
            store_codes();
            drain_exact<kF16>(ws, qlen, lane, blk, wt, tc_out, kv_heads);
            qlen = 0;
            if (kTokenCodes) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the patches have been applied
                unsigned* p = tc_out + (static_cast<size_t>(pend_tile) * 32 + lr) * 4 + half * 2;
                pend_cw.x = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                pend_cw.y = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // consumed here, so that the wait for these two loads stays on this rare path
                asm volatile("" : "+v"(pend_cw.x), "+v"(pend_cw.y));
            }
        };

        // One tile.  `kb` holds its keys; as soon as the matrix cores have consumed them the
        // same registers are reloaded with the tile after next (of the next item at the end
        // of this one), so two tiles are in flight per wave for most of the time without a
        // third buffer.  The reload is unconditional: one skipped on some path would make
        // the compiler wait for everything outstanding.
        // Without token codes there are sixteen registers to spare, and the weight fragments of the first step
        // of a tile stay in them for the whole kernel: no tile then starts with a wait for LDS, and an eighth of
        // the LDS reads is gone.  With token codes the fragments are requested first thing in a tile, ahead of
        // the wait for the keys and of their norms.
        constexpr bool kResidentFirst = !kTokenCodes;
        u32x4 wf_first[4];
        if (kResidentFirst) {
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                wf_first[nb] = *reinterpret_cast<const u32x4*>(&wt[(nb * 32 + lr) * kWtStride + half * 8]);
            }
        }
        auto process = [&](u32x4 (&kb)[8], unsigned tile) {
            u32x4 wf[2][4];
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                if (kResidentFirst) { wf[0][nb] = wf_first[nb]; }
                else { wf[0][nb] = *reinterpret_cast<const u32x4*>(&wt[(nb * 32 + lr) * kWtStride + half * 8]); }
            }
            __builtin_amdgcn_sched_barrier(0);
            store_codes();

            // ||x||^2 of vector lr, in four partial sums: one chain of thirty-two dependent dot instructions
            // would leave the wave waiting on each one's latency
            float xp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned e = kb[ks][j];
                    xp[j] = dot2_self<kF16>(e, xp[j]);
                }
            }
            float xn2 = (xp[0] + xp[1]) + (xp[2] + xp[3]);
            xn2 += __shfl_xor(xn2, 32, 64);
            const float sx = sqrtf(xn2);

            f32x16 acc[4];
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
                for (int i = 0; i < 16; ++i) { acc[nb][i] = 0.0f; }
            }
            // the weight fragments of a step are read from LDS while the matrix instructions of the step before run
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const u32x4 kf = kb[ks];
                if (ks < 7) {
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) {
                        wf[(ks + 1) & 1][nb] = *reinterpret_cast<const u32x4*>(&wt[(nb * 32 + lr) * kWtStride + half * 8 + (ks + 1) * 16]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    acc[nb] = mfma_32x32x16<kF16>(wf[ks & 1][nb], kf, acc[nb]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            {
                const unsigned t2 = tile + 2;
                const bool over = t2 >= n_tiles;
                load_tile(kb, over ? next_blk : blk, over ? (chain ? t2 - n_tiles : n_tiles - 1) : t2);
            }
            __builtin_amdgcn_sched_barrier(0);

            // sign bits -> compact words: bit 16*(nb%2) + i of pair nb/2 is accumulator i of block nb
            unsigned pair[2];
            unsigned long long doubt[4];
#pragma unroll
            for (int wp = 0; wp < 2; ++wp) {
                unsigned wbits = 0u;
#pragma unroll
                for (int sub = 1; sub >= 0; --sub) {
                    const int nb = 2 * wp + sub;
                    // (the minimum starts at the largest finite value and the test is "not at or above", so that a
                    // bound of infinity or NaN - a key with a component beyond 1e19, infinite or NaN, whose sums
                    // may have overflowed on the way - flags the column block whatever the results are)
                    float mn = 0x1.fffffep+127f;
#pragma unroll
                    for (int i = 15; i >= 0; --i) {
                        wbits = __builtin_amdgcn_alignbit(wbits, __float_as_uint(acc[nb][i]), 31);
                        mn = __builtin_fminf(mn, __builtin_fabsf(acc[nb][i]));
                    }
                    doubt[nb] = __ballot(!(mn >= sw[nb] * sx));
                }
                pair[wp] = wbits;
            }
            planes_add(planes01, pair[0]);
            planes_add(planes23, pair[1]);
            ++pending;

            if (kTokenCodes) {
                // This tile's code words: 32 vectors x 16 B, contiguous.  A lane holds the lower (half 0)
                // or upper (half 1) sixteen bits of all four words of its vector; lane lr keeps words 0-1,
                // lane lr+32 words 2-3 (stored at the start of the next tile, see store_codes).  One
                // exchange between the lane halves brings both parts of a lane's two words together:
                // lower lanes then hold (own pair 0, partner's pair 0), upper lanes (partner's pair 1,
                // own pair 1), lower sixteen columns first either way.
                const auto both = __builtin_amdgcn_permlane32_swap(pair[0], pair[1], false, false);
                pend_cw.x = __builtin_amdgcn_perm(both[1], both[0], 0x05040100u);
                pend_cw.y = __builtin_amdgcn_perm(both[1], both[0], 0x07060302u);
                pend_tile = tile;
            }

            // second look, only at the flagged column blocks (with Gaussian keys about one block
            // per tile is flagged, so all four flags are tested with one branch first): the sign of
            // |acc| - bound marks the doubtful ones of a lane's sixteen results (one sub and one
            // v_alignbit each, no LDS, no branches), and the lanes that have any pop them into the
            // queue.  The provisional bit of an entry is read back from the packed sign word.
            if (doubt[0] | doubt[1] | doubt[2] | doubt[3]) {
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    if (doubt[nb]) {
                        const float bound = sw[nb] * sx;     // an all-zero key has bound 0: nothing is below it
                        unsigned mask = 0u;
#pragma unroll
                        for (int i = 15; i >= 0; --i) {
                            mask = __builtin_amdgcn_alignbit(mask, __float_as_uint(__builtin_fabsf(acc[nb][i]) - bound), 31);
                        }
                        if (!(bound < __builtin_inff())) { mask = 0xffffu; }    // no finite bound: all sixteen are redone
                        const unsigned signs = pair[nb >> 1] >> (16 * (nb & 1));
                        unsigned long long um = __ballot(mask != 0u);
                        while (um) {
                            if (qlen + 64 > kQueueCap) { drain_queue(); }
                            if (mask) {
                                const unsigned i = static_cast<unsigned>(__builtin_ctz(mask));
                                mask &= mask - 1u;
                                const unsigned col = nb * 32 + half * 16 + i;
                                ws.queue[qlen + static_cast<int>(lanes_below(um))] =
                                    ((tile * 32 + lr) << 8) | (col << 1) | ((signs >> i) & 1u);
                            }
                            qlen += __popcll(um);
                            um = __ballot(mask != 0u);
                        }
                    }
                }
            }

            if (pending == kFlushTiles) {
                flush_planes();
                pending = 0;
            }
        };

        if (!prefetched) {
            load_tile(k_a, blk, 0);
            load_tile(k_b, blk, min(1u, n_tiles - 1));
        }
        prefetched = chain;
        unsigned tile = 0;
#pragma unroll 1
        for (; tile + 1 < n_tiles; tile += 2) {
            process(k_a, tile);
            process(k_b, tile + 1);
        }
        if (tile < n_tiles) {
            process(k_a, tile);
            // an odd tile count leaves the next item's tile 0 in k_b and its tile 1 in k_a
            if (chain) {
#pragma unroll
                for (int ks = 0; ks < 8; ++ks) { const u32x4 t = k_a[ks]; k_a[ks] = k_b[ks]; k_b[ks] = t; }
            }
        }
        store_codes();
        if (qlen > 0) { drain_exact<kF16>(ws, qlen, lane, blk, wt, tc_out, kv_heads); }
        flush_planes_last();

        // ---- block summaries
        // (LDS operations of one wave complete in order; no barrier is needed inside the wave)
        short* cs = colsum_out + (static_cast<int64_t>(l) * cs_layer_stride + static_cast<int64_t>(slot) * kv_heads * kBits);
        unsigned* bc = block_codes + (static_cast<int64_t>(l) * bc_layer_stride + static_cast<int64_t>(slot) * kv_heads * 4);
        for (unsigned h = 0; h < kv_heads; ++h) {
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                const int col = part * 64 + lane;
                const int n_ones = ws.colsum[h][col];
                const int sgn = 2 * n_ones - static_cast<int>(tokens);
                cs[h * kBits + col] = static_cast<short>(sgn);
                const unsigned long long m = __ballot(sgn > 0);
                if (lane == 0) {
                    bc[h * 4 + part * 2] = static_cast<unsigned>(m);
                    bc[h * 4 + part * 2 + 1] = static_cast<unsigned>(m >> 32);
                }
            }
        }
    }
}

// Query side, one workgroup of four waves per (request, layer); wave w projects every vector onto weight
// columns 32w .. 32w+31 on the matrix cores.  The vectors are the request's q_heads query rows (32 per
// tile) and the kv_heads group-mean queries (fp32 sequential adds * (1/g), the scoring path's own mean).
// A mean is an fp32 number, not a bf16 one: it is cut exactly into three bf16 terms (leading 8 bits, the
// next 8, the rest), which become rows h, 8+h and 16+h of one more tile; those three rows of a column are
// registers i, i+4, i+8 of the same lane and are added there.  Only signs are kept, and they must be the
// signs of the exactly accumulated products: a result whose magnitude is below
// 2^-15 * (largest ||x|| of the tile) * ||w_col|| - more than the fp32 accumulation can be off by - is redone
// by its lane in fp64, d ascending (a product of an fp32 and a bf16 value is exact in fp64), every lane
// working on one of its own results at a time.  A tile whose vectors are all tiny (norm below 2^-60, where
// bf16 subnormals and the bound itself lose bits) is redone whole.  Query rows are the A operand and weights
// the B operand, so a lane holds one weight column and 16 vectors, and a ballot over the lanes is a vector's
// 32-bit code word.  The weights sit in LDS in their own [d][column] order (a lane reads its column two
// bytes at a time, neighbours in neighbouring banks); the means are formed once per workgroup, a 16-byte
// piece per thread, and parked in LDS as their three terms.
// grid: x = request, y = layer; 256 threads
constexpr int kMaxQHeads = 128;
constexpr int kQueryThreads = 256;
constexpr int kMeanStride = kDim + 8;                    // bf16 elements per staged term row (272 B)

struct __attribute__((aligned(16))) QueryLds {
    unsigned short w[kDim * kBits];                      // [d][column]
    unsigned short mean[3][kMaxHeads][kMeanStride];      // [term][kv head][d]
    float mean_max2[2];                                  // largest squared norm of the means staged by waves 0 and 1
};

static_assert(sizeof(QueryLds::mean) >= kMaxHeads * kDim * sizeof(float), "the term area also holds the means as fp32 rows");

__device__ __forceinline__ float wave_max32(float m)
{
#pragma unroll
    for (int d = 16; d >= 1; d >>= 1) { m = fmaxf(m, __shfl_xor(m, d, 64)); }
    return m;
}

template <bool kF16>
__device__ __forceinline__ void widen8(const u32x4 v, float (&x)[8])
{
    const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { x[2 * j] = widen_lo<kF16>(w[j]); x[2 * j + 1] = widen_hi<kF16>(w[j]); }
}

// acc += x[0..7] . W[d0 .. d0+7][col], d ascending (exact products, fp64 sums: the oracle's arithmetic)
template <bool kF16>
__device__ __forceinline__ double dot8_exact(const float (&x)[8], const unsigned short* w_s, unsigned d0, unsigned col, double acc)
{
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float wf = widen_lo<kF16>(static_cast<unsigned>(w_s[(d0 + j) * kBits + col]));
        acc += static_cast<double>(x[j]) * static_cast<double>(wf);
    }
    return acc;
}

// exact sign of a query row . column: the row is fetched in four groups of four 16-byte pieces
template <bool kF16>
__device__ __forceinline__ bool row_exact_positive(const unsigned short* __restrict__ row, const unsigned short* w_s, unsigned col)
{
    double acc = 0.0;
#pragma unroll 1
    for (int c = 0; c < 4; ++c) {
        u32x4 xv[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) { xv[k] = ucm::gload16(row + 32 * c + 8 * k); }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float x[8];
            widen8<kF16>(xv[k], x);
            acc = dot8_exact<kF16>(x, w_s, 32 * c + 8 * k, col, acc);
        }
    }
    return acc > 0.0;
}

// exact sign of a staged group mean . column; (hi + mid) + lo is the mean again, exactly
template <bool kF16>
__device__ __forceinline__ bool mean_exact_positive(const QueryLds& s, unsigned h, unsigned col)
{
    double acc = 0.0;
#pragma unroll 1
    for (int k = 0; k < kDim / 8; ++k) {
        float hi[8], mid[8], lo[8], x[8];
        widen8<kF16>(*reinterpret_cast<const u32x4*>(&s.mean[0][h][8 * k]), hi);
        widen8<kF16>(*reinterpret_cast<const u32x4*>(&s.mean[1][h][8 * k]), mid);
        widen8<kF16>(*reinterpret_cast<const u32x4*>(&s.mean[2][h][8 * k]), lo);
#pragma unroll
        for (int j = 0; j < 8; ++j) { x[j] = (hi[j] + mid[j]) + lo[j]; }
        acc = dot8_exact<kF16>(x, s.w, 8 * k, col, acc);
    }
    return acc > 0.0;
}

// exact sign of an fp32 mean . column (float16 model, several query heads per kv head: the means wait in the
// term area as plain fp32 rows; an fp32 times a float16 value is exact in fp64 as well)
__device__ __forceinline__ bool mean_f32_exact_positive(const QueryLds& s, unsigned h, unsigned col)
{
    const float* m = reinterpret_cast<const float*>(&s.mean[0][0][0]) + h * kDim;
    double acc = 0.0;
#pragma unroll 8
    for (int d = 0; d < kDim; ++d) {
        const float wf = widen_lo<true>(static_cast<unsigned>(s.w[d * kBits + col]));
        acc += static_cast<double>(m[d]) * static_cast<double>(wf);
    }
    return acc > 0.0;
}

// kF16: float16 queries and weights.  With one query head per kv head the "mean" is the row itself, which is its own
// first term.  An fp32 mean of several float16 rows does not split into float16 terms exactly (its low bits fall
// below what float16 can hold), so these few means (kv_heads per request) skip the matrix cores: they are kept in
// fp32 and every one of their signs is taken the exact way.
template <bool kF16>
__global__ __launch_bounds__(kQueryThreads, 4) void hash_query_kernel(
    const unsigned short* __restrict__ q, int64_t q_layer_stride, const int32_t* __restrict__ q_rows,
    unsigned q_heads, unsigned kv_heads, const unsigned short* __restrict__ w, unsigned n_req,
    unsigned* __restrict__ q_codes /*[L][n_req][q_heads][4]*/, short* __restrict__ q_sum /*[L][n_req][128]*/,
    unsigned* __restrict__ qbar_codes /*[L][n_req][kv_heads][4]*/)
{
    __shared__ QueryLds s;
    const unsigned r = blockIdx.x, l = blockIdx.y;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned half = lane >> 5, lr32 = lane & 31;
    const unsigned col = wave * 32 + lr32;               // the weight column this lane ends up with
    // a row index that came from device memory is followed only inside the layer's query block
    const int64_t q_row = q_rows ? static_cast<int64_t>(q_rows[r]) : r;
    if (q_rows && (q_row < 0 || (q_row + 1) * q_heads * kDim > q_layer_stride)) { return; }  // (the whole workgroup)
    const unsigned short* qp = q + static_cast<int64_t>(l) * q_layer_stride + q_row * q_heads * kDim;
    const size_t lrq = static_cast<size_t>(l) * n_req + r;
    const unsigned g = q_heads / kv_heads;
    const float inv = 1.0f / static_cast<float>(g);

    // ---- staging: the weights as they are, and the means' three terms (thread = head, 16-byte piece)
    {
        u32x4 wv[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) { wv[k] = ucm::gload16(w + (k * kQueryThreads + threadIdx.x) * 8); }
        const unsigned h = threadIdx.x >> 4, piece = threadIdx.x & 15;
        float nx2 = 0.0f;
        if (h < kv_heads) {
            const unsigned short* first = qp + (h * g) * kDim + 8 * piece;
            float x[8];
            widen8<kF16>(ucm::gload16(first), x);
#pragma unroll 4
            for (unsigned rr = 1; rr < g; ++rr) {
                float y[8];
                widen8<kF16>(ucm::gload16(first + rr * kDim), y);
#pragma unroll
                for (int j = 0; j < 8; ++j) { x[j] = x[j] + y[j]; }
            }
            unsigned term[3][8];
            float xmean[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xm = g != 1 ? x[j] * inv : x[j];
                xmean[j] = xm;
                if (kF16) {                                                   // (g == 1: xm is a float16 value)
                    term[0][j] = __builtin_bit_cast(unsigned short, static_cast<_Float16>(xm));
                    term[1][j] = term[2][j] = 0u;
                } else {
                    const float hi = __uint_as_float(__float_as_uint(xm) & 0xffff0000u);
                    const float r1 = xm - hi;                                 // exact: the trailing bits of xm
                    const float mid = __uint_as_float(__float_as_uint(r1) & 0xffff0000u);
                    const float lo = r1 - mid;                                // exact, at most 8 significant bits
                    term[0][j] = __float_as_uint(hi) >> 16;
                    term[1][j] = __float_as_uint(mid) >> 16;
                    term[2][j] = __float_as_uint(lo) >> 16;
                }
                nx2 = nx2 + xm * xm;
            }
            if (kF16 && g != 1) {
                float* m = reinterpret_cast<float*>(&s.mean[0][0][0]) + h * kDim + 8 * piece;
#pragma unroll
                for (int j = 0; j < 8; ++j) { m[j] = xmean[j]; }
            } else {
#pragma unroll
                for (int p = 0; p < 3; ++p) {
                    u32x4 packed;
#pragma unroll
                    for (int j = 0; j < 4; ++j) { packed[j] = term[p][2 * j] | (term[p][2 * j + 1] << 16); }
                    *reinterpret_cast<u32x4*>(&s.mean[p][h][8 * piece]) = packed;
                }
            }
        }
        if (wave < 2) {                                  // (waves 0 and 1 hold the at most eight heads)
#pragma unroll
            for (int d = 8; d >= 1; d >>= 1) { nx2 += __shfl_xor(nx2, d, 64); }      // a head's 16 pieces
            nx2 = fmaxf(nx2, __shfl_xor(nx2, 16, 64));
            nx2 = fmaxf(nx2, __shfl_xor(nx2, 32, 64));
            if (lane == 0) { s.mean_max2[wave] = nx2; }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) { *reinterpret_cast<u32x4*>(&s.w[(k * kQueryThreads + threadIdx.x) * 8]) = wv[k]; }
    }
    __syncthreads();

    // B operand: step ks covers dims 16ks .. 16ks+15, this lane holds the eight of its half for its column
    u32x4 wb[8];
    float nw2 = 0.0f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        const unsigned short* wp = &s.w[(16 * ks + 8 * half) * kBits + col];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            wb[ks][j] = static_cast<unsigned>(wp[(2 * j) * kBits]) | (static_cast<unsigned>(wp[(2 * j + 1) * kBits]) << 16);
        }
        nw2 = norm2_acc<kF16>(wb[ks], nw2);
    }
    nw2 += __shfl_xor(nw2, 32, 64);                      // the column's squared norm

    // ---- the query rows, 32 per tile
    int sum = 0;
    for (unsigned t0 = 0; t0 < q_heads; t0 += 32) {
        const unsigned m_in = t0 + lr32;                 // the row this lane feeds
        u32x4 xa[8];
        float nx2 = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            if (m_in < q_heads) { xa[ks] = ucm::gload16(qp + m_in * kDim + 16 * ks + 8 * half); }
            else { xa[ks] = u32x4{0u, 0u, 0u, 0u}; }
            nx2 = norm2_acc<kF16>(xa[ks], nx2);
        }
        nx2 += __shfl_xor(nx2, 32, 64);
        const float max2 = wave_max32(nx2);
        const bool all_exact = (max2 > 0.0f && !(max2 >= 0x1p-120f)) || !(max2 < __builtin_inff());   // tiny norms, or none that is finite
        const float bound = sqrtf(kTau2 * max2) * sqrtf(nw2) * 1.01f;
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) { acc[i] = 0.0f; }
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            acc = mfma_32x32x16<kF16>(xa[ks], wb[ks], acc);
        }
        // result register i is row t0 + 8*(i/4) + 4*half + i%4
        unsigned positive = 0, redo = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const bool valid = t0 + 8 * (i >> 2) + 4 * half + (i & 3) < q_heads;
            if (acc[i] > 0.0f) { positive |= 1u << i; }
            if (valid && (all_exact || !(fabsf(acc[i]) >= bound))) { redo |= 1u << i; }
        }
        while (redo) {
            const unsigned i = static_cast<unsigned>(__builtin_ctz(redo));
            redo &= redo - 1;
            const unsigned m = t0 + 8 * (i >> 2) + 4 * half + (i & 3);
            const bool pos = row_exact_positive<kF16>(qp + m * kDim, s.w, col);
            positive = (positive & ~(1u << i)) | (static_cast<unsigned>(pos) << i);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const unsigned m = t0 + 8 * (i >> 2) + 4 * half + (i & 3);
            const bool valid = m < q_heads;
            const bool pos = valid && ((positive >> i) & 1u);
            const unsigned long long mask = __ballot(pos);
            if (valid) {
                sum += pos ? 1 : -1;
                if (lr32 == 0) { q_codes[(lrq * q_heads + m) * 4 + wave] = static_cast<unsigned>(half ? mask >> 32 : mask); }
            }
        }
    }
    sum += __shfl_xor(sum, 32, 64);
    if (half == 0) { q_sum[lrq * kBits + col] = static_cast<short>(sum); }

    // ---- the group means
    if (kF16 && g != 1) {
#pragma unroll 1
        for (unsigned i = 0; i < 4; ++i) {
            const unsigned h = 4 * half + i;
            const bool valid = h < kv_heads;
            const bool pos = valid && mean_f32_exact_positive(s, h, col);
            const unsigned long long mask = __ballot(pos);
            if (valid && lr32 == 0) {
                qbar_codes[(lrq * kv_heads + h) * 4 + wave] = static_cast<unsigned>(half ? mask >> 32 : mask);
            }
        }
    } else {                                             // row 8*term + h of the tile is that term of head h's mean
        const unsigned term = lr32 >> 3, h_in = lr32 & 7;
        const bool feeds = term < 3 && h_in < kv_heads;
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) { acc[i] = 0.0f; }
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            u32x4 xa = u32x4{0u, 0u, 0u, 0u};
            if (feeds) { xa = *reinterpret_cast<const u32x4*>(&s.mean[term][h_in][16 * ks + 8 * half]); }
            acc = mfma_32x32x16<kF16>(xa, wb[ks], acc);
        }
        const float max2 = fmaxf(s.mean_max2[0], s.mean_max2[1]);
        const bool all_exact = (max2 > 0.0f && !(max2 >= 0x1p-120f)) || !(max2 < __builtin_inff());   // tiny norms, or none that is finite
        const float bound = sqrtf(kTau2 * max2) * sqrtf(nw2) * 1.01f;
        unsigned positive = 0, redo = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float t = (acc[i] + acc[i + 4]) + acc[i + 8];      // the three terms of head 4*half + i
            if (t > 0.0f) { positive |= 1u << i; }
            if (4 * half + i < kv_heads && (all_exact || !(fabsf(t) >= bound))) { redo |= 1u << i; }
        }
        while (redo) {
            const unsigned i = static_cast<unsigned>(__builtin_ctz(redo));
            redo &= redo - 1;
            const bool pos = mean_exact_positive<kF16>(s, 4 * half + i, col);
            positive = (positive & ~(1u << i)) | (static_cast<unsigned>(pos) << i);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned h = 4 * half + i;
            const bool valid = h < kv_heads;
            const unsigned long long mask = __ballot(valid && ((positive >> i) & 1u));
            if (valid && lr32 == 0) {
                qbar_codes[(lrq * kv_heads + h) * 4 + wave] = static_cast<unsigned>(half ? mask >> 32 : mask);
            }
        }
    }
}

__device__ __forceinline__ float half_round(float x)
{
    // round-to-nearest-even to fp16 and back (overflow -> inf), the reference's score dtype
    return static_cast<float>(static_cast<_Float16>(x));
}

typedef short i16x8 __attribute__((ext_vector_type(8)));

// Blocks of a request whose rows lie inside the summary tables; a request outside them (its descriptors live in
// device memory, where the host cannot check them) counts none and is not scored.
__device__ __forceinline__ int seg_blocks(int off, int len, int64_t rows)
{
    const int n = max(len, 0);
    return off >= 0 && static_cast<int64_t>(off) + n <= rows ? n : 0;
}

// Integer block scores <sum_i u(q_i), sum_h S[h]>.  Sixteen lanes share one block:
// lane j owns bits 8j..8j+7 of the 128-entry column-sum row (one 16-byte load per
// kv head, 256 contiguous bytes per 16 lanes); a 16-lane shuffle reduction adds
// the partial scores.  Requests are found by a scan of the segment lengths
// (they are few; rows are many).
// grid: x = 16 rows of the ragged batch (dense numbering), y = layer; 256 threads
__global__ __launch_bounds__(256) void hash_score_kernel(
    const short* __restrict__ q_sum, const short* __restrict__ colsum, int64_t cs_layer_stride,
    const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len,
    unsigned n_req, unsigned kv_heads, float* __restrict__ scores, int64_t scores_layer_stride, int round_fp16, int64_t rows)
{
    const unsigned l = blockIdx.y;
    const unsigned sub = threadIdx.x & 15;
    int dense = blockIdx.x * 16 + (threadIdx.x >> 4);
    int r = -1, local = 0;
    for (unsigned i = 0; i < n_req; ++i) {
        const int n = seg_blocks(seg_off[i], seg_len[i], rows);
        if (dense < n) { r = static_cast<int>(i); local = dense; break; }
        dense -= n;
    }
    int score = 0;
    int64_t row = 0;
    if (r >= 0) {
        row = static_cast<int64_t>(seg_off[r]) + local;
        const size_t lr = static_cast<size_t>(l) * n_req + r;
        const short* cs = colsum + static_cast<int64_t>(l) * cs_layer_stride + row * kv_heads * kBits + sub * 8;
        const i16x8 qv = *reinterpret_cast<const i16x8*>(q_sum + lr * kBits + sub * 8);
        int s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        // every head's load is issued before the first sum (a loop over a head count known only at run time waits
        // for each load in turn: eight memory round trips per block instead of one; 64 -> 60 us for 32 layers x 5294
        // blocks.  Two or four blocks per group of sixteen lanes, with a search for their requests that cannot leave
        // early, took 68 and 87 us.)
        i16x8 v[kMaxHeads];
#pragma unroll
        for (unsigned h = 0; h < kMaxHeads; ++h) {
            v[h] = *reinterpret_cast<const i16x8*>(cs + (h < kv_heads ? h : 0u) * kBits);
        }
#pragma unroll
        for (unsigned h = 0; h < kMaxHeads; ++h) {
            if (h < kv_heads) {
#pragma unroll
                for (int k = 0; k < 8; ++k) { s[k] += v[h][k]; }
            }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) { score += static_cast<int>(qv[k]) * s[k]; }
    }
    score += __shfl_xor(score, 8, 16);
    score += __shfl_xor(score, 4, 16);
    score += __shfl_xor(score, 2, 16);
    score += __shfl_xor(score, 1, 16);
    if (r >= 0 && sub == 0) {
        float f = static_cast<float>(score);
        if (round_fp16) { f = half_round(f); }
        scores[static_cast<int64_t>(l) * scores_layer_stride + row] = f;
    }
}

// Block-code score: sum over kv heads of (bits - hamming(code of the group-mean query, majority code of the
// block)).  128 bytes per block, so what counts is the number of requests in flight,
// not arithmetic.  Eight lanes share a block, lane h holding kv head h's 128-bit majority code (one
// 16-byte load); a thread handles four blocks, 32 apart, whose loads are issued together; the owning
// request of a block is found without an early exit, so the segment lengths arrive in a few wide scalar
// loads.
// grid: x = 128 rows of the ragged batch (dense numbering), y = layer; 256 threads
constexpr int kCodeBlocksPerGroup = 128;

__global__ __launch_bounds__(256) void hash_code_score_kernel(
    const unsigned* __restrict__ qbar_codes, const unsigned* __restrict__ block_codes, int64_t bc_layer_stride,
    const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len, unsigned n_req, unsigned kv_heads,
    float* __restrict__ scores, int64_t scores_layer_stride, int round_fp16, int64_t rows)
{
    const unsigned l = blockIdx.y, h = threadIdx.x & 7;
    int req[4];
    int64_t row[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) { req[u] = -1; row[u] = 0; }
    const int first = blockIdx.x * kCodeBlocksPerGroup + (threadIdx.x >> 3);
    int base = 0;
    for (unsigned i = 0; i < n_req; ++i) {
        const int off = seg_off[i], n = seg_blocks(off, seg_len[i], rows);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int dense = first + 32 * u;
            if (req[u] < 0 && dense < base + n) { req[u] = static_cast<int>(i); row[u] = static_cast<int64_t>(off) + (dense - base); }
        }
        base += n;
    }
    u32x4 bc[4], qc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        bc[u] = qc[u] = u32x4{0u, 0u, 0u, 0u};
        if (req[u] >= 0 && h < kv_heads) {
            bc[u] = ucm::gload16(block_codes + static_cast<int64_t>(l) * bc_layer_stride + (row[u] * kv_heads + h) * 4);
            qc[u] = ucm::gload16(qbar_codes + ((static_cast<size_t>(l) * n_req + req[u]) * kv_heads + h) * 4);
        }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        int score = 0;
        if (h < kv_heads) {
#pragma unroll
            for (int k = 0; k < 4; ++k) { score += 32 - __popc(bc[u][k] ^ qc[u][k]); }
        }
        score += __shfl_xor(score, 4, 8);
        score += __shfl_xor(score, 2, 8);
        score += __shfl_xor(score, 1, 8);
        if (req[u] >= 0 && h == 0) {
            float f = static_cast<float>(score);
            if (round_fp16) { f = half_round(f); }
            scores[static_cast<int64_t>(l) * scores_layer_stride + row[u]] = f;
        }
    }
}

}  // namespace

namespace {

int hash_encode_blocks(bool f16, const void* const* k_layers, int n_layers, int num_blocks,
                       const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                       int kv_heads, int head_dim, const void* w_bf16, int bits, int rows,
                       uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                       int64_t colsum_layer_stride, uint8_t* block_codes,
                       int64_t block_codes_layer_stride, int workgroups, ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0, "ucm_hash_encode_blocks: n=%d", n);
    UCM_REQUIRE(workgroups >= 0 && workgroups <= (1 << 20), "ucm_hash_encode_blocks: workgroups=%d", workgroups);
    const int encode_groups = workgroups > 0 ? workgroups : 4096;
    if (n == 0) { return UCM_OK; }
    UCM_REQUIRE(k_layers && w_bf16 && colsum && block_codes, "ucm_hash_encode_blocks: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers <= 65535 && num_blocks > 0 && rows > 0 && block_size > 0,
                "ucm_hash_encode_blocks: non-positive shape");
    UCM_SUPPORTED(head_dim == kDim && bits == kBits, "ucm_hash_encode_blocks: head_dim=%d bits=%d (128 and 128)", head_dim, bits);
    UCM_SUPPORTED(kv_heads == 1 || kv_heads == 2 || kv_heads == 4 || kv_heads == 8,
                  "ucm_hash_encode_blocks: kv_heads=%d (1, 2, 4 or 8)", kv_heads);
    UCM_SUPPORTED((block_size * kv_heads) % 32 == 0 && block_size <= 16383,
                  "ucm_hash_encode_blocks: block_size*kv_heads=%d must be a multiple of 32", block_size * kv_heads);
    UCM_REQUIRE(ucm::aligned16(token_codes) && token_codes_layer_stride % 16 == 0,
                "ucm_hash_encode_blocks: token_codes must be 16-byte aligned");
    UCM_REQUIRE(token_codes_layer_stride % 4 == 0 && block_codes_layer_stride % 4 == 0,
                "ucm_hash_encode_blocks: code strides are in bytes and must be multiples of 4");
    // persistent workgroups: about 4096 of them over all layers, each wave stepping through the list
    const int groups = (n + kWaves - 1) / kWaves;
    const int gx = std::min(groups, std::max(1, (encode_groups + n_layers - 1) / n_layers));
#define UCM_HASH_ENCODE_ARGS dim3(gx, n_layers), dim3(kThreads), 0, ucm::as_stream(stream), k_layers, block_ids, slots, \
        static_cast<unsigned>(num_blocks), static_cast<unsigned>(n), static_cast<unsigned>(rows),                        \
        static_cast<unsigned>(block_size), static_cast<unsigned>(kv_heads), static_cast<const unsigned short*>(w_bf16),  \
        reinterpret_cast<unsigned*>(token_codes), token_codes_layer_stride / 4, colsum, colsum_layer_stride,             \
        reinterpret_cast<unsigned*>(block_codes), block_codes_layer_stride / 4
    if (f16) {
        if (token_codes) { hipLaunchKernelGGL((hash_encode_blocks_kernel<true, true>), UCM_HASH_ENCODE_ARGS); }
        else { hipLaunchKernelGGL((hash_encode_blocks_kernel<false, true>), UCM_HASH_ENCODE_ARGS); }
    } else {
        if (token_codes) { hipLaunchKernelGGL((hash_encode_blocks_kernel<true, false>), UCM_HASH_ENCODE_ARGS); }
        else { hipLaunchKernelGGL((hash_encode_blocks_kernel<false, false>), UCM_HASH_ENCODE_ARGS); }
    }
#undef UCM_HASH_ENCODE_ARGS
    UCM_LAUNCH_CHECK("ucm_hash_encode_blocks");
}

}  // namespace

extern "C" int ucm_hash_encode_blocks(const void* const* k_layers, int n_layers, int num_blocks,
                                      const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                      int kv_heads, int head_dim, const void* w_bf16, int bits, int rows,
                                      uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                                      int64_t colsum_layer_stride, uint8_t* block_codes,
                                      int64_t block_codes_layer_stride, int workgroups, ucm_stream_t stream)
{
    return hash_encode_blocks(false, k_layers, n_layers, num_blocks, block_ids, slots, n, block_size, kv_heads, head_dim, w_bf16,
                              bits, rows, token_codes, token_codes_layer_stride, colsum, colsum_layer_stride, block_codes,
                              block_codes_layer_stride, workgroups, stream);
}

extern "C" int ucm_hash_encode_blocks_f16(const void* const* k_layers, int n_layers, int num_blocks,
                                          const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                          int kv_heads, int head_dim, const void* w_f16, int bits, int rows,
                                          uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                                          int64_t colsum_layer_stride, uint8_t* block_codes,
                                          int64_t block_codes_layer_stride, int workgroups, ucm_stream_t stream)
{
    return hash_encode_blocks(true, k_layers, n_layers, num_blocks, block_ids, slots, n, block_size, kv_heads, head_dim, w_f16,
                              bits, rows, token_codes, token_codes_layer_stride, colsum, colsum_layer_stride, block_codes,
                              block_codes_layer_stride, workgroups, stream);
}


namespace {

int hash_encode_queries(bool f16, const void* q_bf16, int64_t q_layer_stride, const int32_t* q_rows,
                        int n_req, int n_layers, int q_heads, int kv_heads, int head_dim,
                        const void* w_bf16, int bits, uint8_t* q_codes, int16_t* q_sum,
                        uint8_t* qbar_codes, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req >= 0 && n_layers > 0 && n_layers <= 65535, "ucm_hash_encode_queries: n_req=%d n_layers=%d", n_req, n_layers);
    if (n_req == 0) { return UCM_OK; }
    UCM_REQUIRE(q_bf16 && w_bf16 && q_codes && q_sum && qbar_codes, "ucm_hash_encode_queries: null pointer");
    UCM_SUPPORTED(head_dim == kDim && bits == kBits, "ucm_hash_encode_queries: head_dim=%d bits=%d (128 and 128)", head_dim, bits);
    UCM_REQUIRE(kv_heads > 0 && q_heads >= kv_heads && q_heads % kv_heads == 0,
                "ucm_hash_encode_queries: q_heads=%d kv_heads=%d", q_heads, kv_heads);
    UCM_REQUIRE(!q_rows || q_layer_stride >= static_cast<int64_t>(q_heads) * head_dim,
                "ucm_hash_encode_queries: with q_rows, q_layer_stride=%lld bounds the rows and must hold at least one",
                static_cast<long long>(q_layer_stride));
    UCM_SUPPORTED(q_heads <= kMaxQHeads && kv_heads <= kMaxHeads, "ucm_hash_encode_queries: q_heads=%d kv_heads=%d (at most %d and %d)",
                  q_heads, kv_heads, kMaxQHeads, kMaxHeads);
#define UCM_HASH_QUERY_ARGS dim3(n_req, n_layers), dim3(kQueryThreads), 0, ucm::as_stream(stream),                    \
        static_cast<const unsigned short*>(q_bf16), q_layer_stride, q_rows, static_cast<unsigned>(q_heads),          \
        static_cast<unsigned>(kv_heads), static_cast<const unsigned short*>(w_bf16), static_cast<unsigned>(n_req),   \
        reinterpret_cast<unsigned*>(q_codes), q_sum, reinterpret_cast<unsigned*>(qbar_codes)
    if (f16) { hipLaunchKernelGGL(hash_query_kernel<true>, UCM_HASH_QUERY_ARGS); }
    else { hipLaunchKernelGGL(hash_query_kernel<false>, UCM_HASH_QUERY_ARGS); }
#undef UCM_HASH_QUERY_ARGS
    UCM_LAUNCH_CHECK("ucm_hash_encode_queries");
}

}  // namespace

extern "C" int ucm_hash_encode_queries(const void* q_bf16, int64_t q_layer_stride, const int32_t* q_rows,
                                       int n_req, int n_layers, int q_heads, int kv_heads, int head_dim,
                                       const void* w_bf16, int bits, uint8_t* q_codes, int16_t* q_sum,
                                       uint8_t* qbar_codes, ucm_stream_t stream)
{
    return hash_encode_queries(false, q_bf16, q_layer_stride, q_rows, n_req, n_layers, q_heads, kv_heads, head_dim, w_bf16, bits,
                               q_codes, q_sum, qbar_codes, stream);
}

extern "C" int ucm_hash_encode_queries_f16(const void* q_f16, int64_t q_layer_stride, const int32_t* q_rows,
                                           int n_req, int n_layers, int q_heads, int kv_heads, int head_dim,
                                           const void* w_f16, int bits, uint8_t* q_codes, int16_t* q_sum,
                                           uint8_t* qbar_codes, ucm_stream_t stream)
{
    return hash_encode_queries(true, q_f16, q_layer_stride, q_rows, n_req, n_layers, q_heads, kv_heads, head_dim, w_f16, bits,
                               q_codes, q_sum, qbar_codes, stream);
}


extern "C" int ucm_hash_score_blocks(int mode, const int16_t* q_sum, const uint8_t* qbar_codes,
                                     const int16_t* colsum, int64_t colsum_layer_stride,
                                     const uint8_t* block_codes, int64_t block_codes_layer_stride,
                                     int64_t rows, const int32_t* seg_off, const int32_t* seg_len, int n_req,
                                     int64_t total_blocks, int n_layers, int kv_heads, int bits, float* scores,
                                     int64_t scores_layer_stride, int round_fp16, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req >= 0 && total_blocks >= 0 && n_layers > 0 && n_layers <= 65535 && rows >= 0,
                "ucm_hash_score_blocks: n_req=%d n_layers=%d rows=%lld", n_req, n_layers, static_cast<long long>(rows));
    UCM_REQUIRE(n_layers == 1 || scores_layer_stride >= rows, "ucm_hash_score_blocks: scores_layer_stride=%lld < rows=%lld",
                static_cast<long long>(scores_layer_stride), static_cast<long long>(rows));
    if (n_req == 0 || total_blocks == 0) { return UCM_OK; }
    UCM_REQUIRE(mode == 0 || mode == 1, "ucm_hash_score_blocks: mode=%d", mode);
    UCM_REQUIRE(seg_off && seg_len && scores, "ucm_hash_score_blocks: null pointer");
    UCM_REQUIRE(mode == 0 ? (q_sum && colsum) : (qbar_codes && block_codes), "ucm_hash_score_blocks: null operand for this mode");
    UCM_SUPPORTED(bits == kBits && kv_heads >= 1 && kv_heads <= kMaxHeads, "ucm_hash_score_blocks: bits=%d kv_heads=%d", bits, kv_heads);
    const unsigned gx = static_cast<unsigned>((total_blocks + 15) / 16);
    hipStream_t s = ucm::as_stream(stream);
    if (mode == 0) {
        hipLaunchKernelGGL(hash_score_kernel, dim3(gx, n_layers), dim3(256), 0, s, q_sum, colsum, colsum_layer_stride,
                           seg_off, seg_len, static_cast<unsigned>(n_req), static_cast<unsigned>(kv_heads), scores,
                           scores_layer_stride, round_fp16, rows);
    } else {
        UCM_REQUIRE(ucm::aligned16(qbar_codes) && ucm::aligned16(block_codes) && block_codes_layer_stride % 16 == 0,
                    "ucm_hash_score_blocks: codes must be 16-byte aligned");
        const unsigned gc = static_cast<unsigned>((total_blocks + kCodeBlocksPerGroup - 1) / kCodeBlocksPerGroup);
        hipLaunchKernelGGL(hash_code_score_kernel, dim3(gc, n_layers), dim3(256), 0, s,
                           reinterpret_cast<const unsigned*>(qbar_codes), reinterpret_cast<const unsigned*>(block_codes),
                           block_codes_layer_stride / 4, seg_off, seg_len, static_cast<unsigned>(n_req),
                           static_cast<unsigned>(kv_heads), scores, scores_layer_stride, round_fp16, rows);
    }
    UCM_LAUNCH_CHECK("ucm_hash_score_blocks");
}
