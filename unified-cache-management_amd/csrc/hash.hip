// Hash-code retrieval (KvComp style): sign-random-projection codes of the keys,
// per-block summaries of those codes, query codes, and integer block scores.
//
// The projection [vectors x 128] . [128 x 128] is the one real contraction on
// the whole retrieval path (128 flop per byte of key), so it runs on the matrix
// cores: v_mfma_f32_32x32x16_bf16, one wave per cache block, 32-vector tiles,
// the weight matrix staged once per workgroup in LDS (transposed, padded rows).
// Only the SIGN of each projection is kept, and it has to be the sign of the
// exactly accumulated dot product (the CPU oracle accumulates in fp64), so
// every result whose magnitude is within the fp32 accumulation error bound
//     |acc| < 2^-15 * ||x|| * ||w_c||
// is queued and redone by one lane in fp64, d ascending; a few bits per ten
// thousand take that path (a one-compare filter with the tile's largest row
// norm flags column blocks; only flagged ones get the per-row look).  The next tile's
// keys are in flight while the current one goes through the matrix cores.
//
// Per cache block the kernel emits: the token codes (LSB-first packing: bit j
// of byte b is column 8b+j), the per-(kv head, bit) column sums over the
// block's tokens S[h][c] = #ones - #zeros, and the majority-vote block code
// (bit c of head h = S[h][c] > 0).  Both block scores used downstream are
// integer functions of these: the reference's sum over all (query head, kv
// head, token) of +-1 inner products equals <sum_i u(q_i), sum_h S[h]>.
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
constexpr float kTau2 = 0x1p-30f;   // (2^-15)^2

__device__ __forceinline__ unsigned lanes_below(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u));
}

__device__ __forceinline__ float bf16_to_f32(unsigned short h) { return __uint_as_float(static_cast<unsigned>(h) << 16); }

struct __attribute__((aligned(16))) WaveScratch {
    float row_norm2[32];
    unsigned queue[kQueueCap];
    float acc_copy[16][64];         // one column block's accumulators, for the second look
    int colsum[kMaxHeads][kBits];   // corrections + final per-head ones counts
};

// Exact sign of x . W[:, col]: fp64 accumulation, d ascending (the oracle's order).
// Both 256-byte rows are fetched with sixteen 16-byte loads issued together, so
// the redo costs one memory latency, not 128 of them.
__device__ __forceinline__ bool exact_positive(const unsigned short* __restrict__ x,
                                               const unsigned short* __restrict__ wt_col)
{
    u32x4 xv[kDim / 8], wv[kDim / 8];
#pragma unroll
    for (int i = 0; i < kDim / 8; ++i) {
        xv[i] = *reinterpret_cast<const u32x4*>(x + i * 8);
        wv[i] = *reinterpret_cast<const u32x4*>(wt_col + i * 8);
    }
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < kDim / 8; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned xa = xv[i][j], wa = wv[i][j];
            acc += static_cast<double>(__uint_as_float(xa << 16)) * static_cast<double>(__uint_as_float(wa << 16));
            acc += static_cast<double>(__uint_as_float(xa & 0xffff0000u)) *
                   static_cast<double>(__uint_as_float(wa & 0xffff0000u));
        }
    }
    return acc > 0.0;
}

// Queued results are redone exactly, 64 at a time, one per lane.  Entries are
// queued after their tile's code words were stored, so the fix goes to memory.
// Kept out of line: it is called from 64 unrolled places and runs rarely.
__device__ __attribute__((noinline)) void drain_exact(WaveScratch& ws, int qlen, int lane,
                                                      const unsigned short* __restrict__ blk,
                                                      const unsigned short* __restrict__ wt,
                                                      unsigned* __restrict__ tc_out, unsigned kv_heads)
{
    // the code words stored by this wave must have reached L2 before they are patched there;
    // waiting for the stores' acknowledgements is enough (a device-scope fence would write back the whole L2)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    for (int base = 0; base < qlen; base += 64) {
        if (base + lane < qlen) {
            const unsigned e = ws.queue[base + lane];
            const unsigned v = e >> 8, col = (e >> 1) & 127u, prov = e & 1u;
            const bool pos = exact_positive(blk + static_cast<size_t>(v) * kDim, &wt[col * kWtStride]);
            if (static_cast<unsigned>(pos) != prov) {
                if (tc_out) { atomicXor(&tc_out[v * 4 + (col >> 5)], 1u << (col & 31)); }
                atomicAdd(&ws.colsum[v % kv_heads][col], pos ? 1 : -1);
            }
        }
    }
}

// grid: x = group of kWaves items (cache blocks), y = layer
__global__ __launch_bounds__(kThreads, 2) void hash_encode_blocks_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned n_items, unsigned rows,
    unsigned tokens, unsigned kv_heads, const unsigned short* __restrict__ w,
    unsigned* __restrict__ token_codes, int64_t tc_layer_stride,
    short* __restrict__ colsum_out, int64_t cs_layer_stride,
    unsigned* __restrict__ block_codes, int64_t bc_layer_stride)
{
    __shared__ __attribute__((aligned(16))) unsigned short wt[kBits * kWtStride];  // wt[col][d]
    __shared__ float w_norm2[kBits];
    __shared__ WaveScratch scratch[kWaves];

    // ---- weights: global [d][col] -> LDS [col][d]
    for (int e = threadIdx.x; e < kDim * kBits; e += kThreads) {
        const int d = e / kBits, c = e - d * kBits;
        wt[c * kWtStride + d] = w[e];
    }
    __syncthreads();
    if (threadIdx.x < kBits) {
        float s = 0.0f;
        for (int d = 0; d < kDim; ++d) {
            const float v = bf16_to_f32(wt[threadIdx.x * kWtStride + d]);
            s = __builtin_fmaf(v, v, s);
        }
        w_norm2[threadIdx.x] = s;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned item = blockIdx.x * kWaves + wave;
    if (item >= n_items) { return; }
    const unsigned id = block_ids ? static_cast<unsigned>(block_ids[item]) : item;
    const unsigned slot = slots ? static_cast<unsigned>(slots[item]) : item;
    if (id >= num_blocks || slot >= rows) { return; }
    const unsigned l = blockIdx.y;
    const unsigned n_vec = tokens * kv_heads;            // vectors of kDim bf16 in the block
    const unsigned short* blk = static_cast<const unsigned short*>(k_layers[l]) +
                                static_cast<size_t>(id) * n_vec * kDim;
    WaveScratch& ws = scratch[wave];
    for (int e = lane; e < kMaxHeads * kBits; e += 64) { (&ws.colsum[0][0])[e] = 0; }

    const int half = lane >> 5, lr = lane & 31;
    int ones[4][4];                                      // [column block][row % 4]: rows of head (half*4 + e) % kv_heads
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
        for (int e = 0; e < 4; ++e) { ones[nb][e] = 0; }
    }
    int qlen = 0;
    unsigned* tc_out = token_codes ? token_codes + (static_cast<int64_t>(l) * tc_layer_stride +
                                                    static_cast<int64_t>(slot) * n_vec * 4) : nullptr;

    auto drain_queue = [&]() {
        drain_exact(ws, qlen, lane, blk, wt, tc_out, kv_heads);
        qlen = 0;
    };

    const unsigned n_tiles = n_vec / 32;
    // A fragments.  The contraction index may be visited in any order as long as A
    // and B agree, so MFMA step ks of lane (row lr, k-half `half`) takes dims
    // half*64 + ks*8 .. +8: a lane's eight 16-byte loads are then one contiguous
    // 128-byte line of vector tile*32 + lr, fetched from L2 once.
    auto load_tile = [&](bf16x8 (&a)[8], unsigned tile) {
        const unsigned short* xrow = blk + (static_cast<size_t>(tile) * 32 + lr) * kDim + half * 64;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) { a[ks] = *reinterpret_cast<const bf16x8*>(xrow + ks * 8); }
    };
    // which ballot carries this lane's row (lanes 0..31 assemble the code words of row `lane`):
    // kept as 16 all-ones / all-zeros masks in vector registers so that no scalar state is tied up
    const int i_sel = ((lr >> 3) << 2) | (lr & 3);
    const bool use_hi = (lr & 4) != 0;
    unsigned sel_mask[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) { sel_mask[i] = i == i_sel ? 0xffffffffu : 0u; }
    float sw[4];                                         // sqrt(tau^2 * ||w_col||^2) for this lane's 4 columns
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) { sw[nb] = sqrtf(kTau2 * w_norm2[nb * 32 + lr]); }

    auto reduce_tile = [&](const bf16x8 (&a)[8], unsigned tile) {
        float ss = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float v = static_cast<float>(a[ks][j]);
                ss = __builtin_fmaf(v, v, ss);
            }
        }
        ss += __shfl_xor(ss, 32, 64);                    // ||x_row||^2, row = lr
        if (half == 0) { ws.row_norm2[lr] = ss; }
        float mx = ss;                                   // largest row norm of the tile: a cheap first filter
#pragma unroll
        for (int d = 16; d >= 1; d >>= 1) { mx = fmaxf(mx, __shfl_xor(mx, d, 64)); }
        const float smx = sqrtf(mx) * 1.0001f;

        f32x16 acc[4];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) { acc[nb][i] = 0.0f; }
        }
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                const bf16x8 b = *reinterpret_cast<const bf16x8*>(&wt[(nb * 32 + lr) * kWtStride + half * 64 + ks * 8]);
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks], b, acc[nb], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);           // keep the weight fragments of later steps out of registers
        }

        // accumulator i of lane (half, lr): row (i/4)*8 + half*4 + i%4, column nb*32 + lr
        unsigned long long doubt[4];                     // per column block: lanes that may need the exact redo
        unsigned words[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            float min_abs = __builtin_inff();
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float v = acc[nb][i];
                const bool pos = v > 0.0f;
                const unsigned long long m = __ballot(pos);
                ones[nb][i & 3] += pos ? 1 : 0;
                min_abs = fminf(min_abs, fabsf(v));
                const unsigned mine = use_hi ? static_cast<unsigned>(m >> 32) : static_cast<unsigned>(m);
                words[nb] |= mine & sel_mask[i];
                if ((i & 3) == 3) { __builtin_amdgcn_sched_barrier(0); }   // consume the ballots before making more
            }
            doubt[nb] = __ballot(min_abs < sw[nb] * smx);
        }
        // this tile's code words: 32 rows x 16 B, contiguous
        if (tc_out && lane < 32) {
            const u32x4 cw = {words[0], words[1], words[2], words[3]};
            *reinterpret_cast<u32x4*>(tc_out + (static_cast<size_t>(tile) * 32 + lane) * 4) = cw;
        }
        // second look, only at the flagged column blocks, with each row's own norm; what
        // stays doubtful is queued for the exact redo.  The block's accumulators go
        // through LDS so that this rare path is one rolled loop with one call site.
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            if (doubt[nb]) {
#pragma unroll
                for (int i = 0; i < 16; ++i) { ws.acc_copy[i][lane] = acc[nb][i]; }
                const float wn = kTau2 * w_norm2[nb * 32 + lr];
#pragma unroll 1
                for (int i = 0; i < 16; ++i) {
                    const int row = (i >> 2) * 8 + half * 4 + (i & 3);
                    const float v = ws.acc_copy[i][lane];
                    const bool unsure = v * v < wn * ws.row_norm2[row];   // strict: an all-zero row is exactly 0
                    const unsigned long long um = __ballot(unsure);
                    if (um) {
                        if (qlen + 64 > kQueueCap) { drain_queue(); }
                        if (unsure) {
                            ws.queue[qlen + static_cast<int>(lanes_below(um))] =
                                ((tile * 32 + row) << 8) | ((nb * 32 + lr) << 1) | (v > 0.0f ? 1u : 0u);
                        }
                        qlen += __popcll(um);
                    }
                }
            }
        }
    };

    bf16x8 a_cur[8], a_nxt[8];
    if (n_tiles > 0) { load_tile(a_cur, 0); }
#pragma unroll 1
    for (unsigned tile = 0; tile < n_tiles; ++tile) {
        if (tile + 1 < n_tiles) { load_tile(a_nxt, tile + 1); }   // in flight during this tile's MFMAs
        reduce_tile(a_cur, tile);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) { a_cur[ks] = a_nxt[ks]; }
    }
    if (qlen > 0) { drain_queue(); }

    // ---- block summaries
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            atomicAdd(&ws.colsum[(half * 4 + e) % kv_heads][nb * 32 + lr], ones[nb][e]);
        }
    }
    // (LDS operations of one wave complete in order; no barrier is needed inside the wave)
    short* cs = colsum_out + (static_cast<int64_t>(l) * cs_layer_stride + static_cast<int64_t>(slot) * kv_heads * kBits);
    unsigned* bc = block_codes + (static_cast<int64_t>(l) * bc_layer_stride + static_cast<int64_t>(slot) * kv_heads * 4);
    for (unsigned h = 0; h < kv_heads; ++h) {
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            const int col = part * 64 + lane;
            const int n_ones = ws.colsum[h][col];
            const int s = 2 * n_ones - static_cast<int>(tokens);
            cs[h * kBits + col] = static_cast<short>(s);
            const unsigned long long m = __ballot(s > 0);
            if (lane == 0) {
                bc[h * 4 + part * 2] = static_cast<unsigned>(m);
                bc[h * 4 + part * 2 + 1] = static_cast<unsigned>(m >> 32);
            }
        }
    }
}

// Query side, one workgroup of 1024 threads per (request, layer): thread
// (bit c, head group hg) projects heads hg, hg+8, ... exactly (fp64, d
// ascending; there are only q_heads*128 such dot products), the +-1 sum over
// all heads is combined through LDS, and each head group also produces the code
// of the group-mean query of kv heads hg, hg+8, ...  W and the request's query
// rows are staged in LDS once.
// grid: x = request, y = layer
constexpr int kQueryGroups = 8;
constexpr int kQueryThreads = kBits * kQueryGroups;
constexpr int kMaxQHeads = 128;

__global__ __launch_bounds__(kQueryThreads) void hash_query_kernel(
    const unsigned short* __restrict__ q, int64_t q_layer_stride, const int32_t* __restrict__ q_rows,
    unsigned q_heads, unsigned kv_heads, const unsigned short* __restrict__ w, unsigned n_req,
    unsigned* __restrict__ q_codes /*[L][n_req][q_heads][4]*/, short* __restrict__ q_sum /*[L][n_req][128]*/,
    unsigned* __restrict__ qbar_codes /*[L][n_req][kv_heads][4]*/)
{
    __shared__ unsigned short w_s[kDim * kBits];            // [d][c]: lanes read consecutive c
    __shared__ unsigned short q_s[kMaxQHeads * kDim];
    __shared__ int part[kQueryGroups][kBits];

    const unsigned r = blockIdx.x, l = blockIdx.y;
    const unsigned c = threadIdx.x % kBits, hg = threadIdx.x / kBits;
    const unsigned short* qp = q + static_cast<int64_t>(l) * q_layer_stride +
                               static_cast<int64_t>(q_rows ? q_rows[r] : r) * q_heads * kDim;
    for (unsigned e = threadIdx.x; e < kDim * kBits; e += kQueryThreads) { w_s[e] = w[e]; }
    for (unsigned e = threadIdx.x; e < q_heads * kDim; e += kQueryThreads) { q_s[e] = qp[e]; }
    __syncthreads();

    const size_t lr = static_cast<size_t>(l) * n_req + r;
    const unsigned g = q_heads / kv_heads;
    int sum = 0;
    for (unsigned i = hg; i < q_heads; i += kQueryGroups) {
        double acc = 0.0;
        for (int d = 0; d < kDim; ++d) {
            acc += static_cast<double>(bf16_to_f32(q_s[i * kDim + d])) * static_cast<double>(bf16_to_f32(w_s[d * kBits + c]));
        }
        const bool pos = acc > 0.0;
        sum += pos ? 1 : -1;
        const unsigned long long m = __ballot(pos);      // a wave covers 64 consecutive bits of one head
        if ((c & 63) == 0) {
            q_codes[(lr * q_heads + i) * 4 + (c >> 6) * 2] = static_cast<unsigned>(m);
            q_codes[(lr * q_heads + i) * 4 + (c >> 6) * 2 + 1] = static_cast<unsigned>(m >> 32);
        }
    }
    part[hg][c] = sum;
    // group-mean query: fp32 sequential adds * (1/g), the scoring path's own mean, then projected exactly
    const float inv = 1.0f / static_cast<float>(g);
    for (unsigned h = hg; h < kv_heads; h += kQueryGroups) {
        double acc = 0.0;
        for (int d = 0; d < kDim; ++d) {
            float m = bf16_to_f32(q_s[(h * g) * kDim + d]);
            for (unsigned j = 1; j < g; ++j) { m = m + bf16_to_f32(q_s[(h * g + j) * kDim + d]); }
            if (g != 1) { m = m * inv; }
            acc += static_cast<double>(m) * static_cast<double>(bf16_to_f32(w_s[d * kBits + c]));
        }
        const unsigned long long mk = __ballot(acc > 0.0);
        if ((c & 63) == 0) {
            qbar_codes[(lr * kv_heads + h) * 4 + (c >> 6) * 2] = static_cast<unsigned>(mk);
            qbar_codes[(lr * kv_heads + h) * 4 + (c >> 6) * 2 + 1] = static_cast<unsigned>(mk >> 32);
        }
    }
    __syncthreads();
    if (hg == 0) {
        int total = 0;
#pragma unroll
        for (int k = 0; k < kQueryGroups; ++k) { total += part[k][c]; }
        q_sum[lr * kBits + c] = static_cast<short>(total);
    }
}

__device__ __forceinline__ float half_round(float x)
{
    // round-to-nearest-even to fp16 and back (overflow -> inf), the reference's score dtype
    return static_cast<float>(static_cast<_Float16>(x));
}

typedef short i16x8 __attribute__((ext_vector_type(8)));

// Integer block scores.  Sixteen lanes share one block: in mode 0 lane j owns
// bits 8j..8j+7 of the 128-entry column-sum row (one 16-byte load per kv head,
// 256 contiguous bytes per 16 lanes), in mode 1 lanes 0..kv_heads*4-1 each own
// one 32-bit word of the block code; a 16-lane DPP-free shuffle reduction adds
// the partial scores.  Requests are found by a scan of the segment lengths
// (they are few; rows are many).
// grid: x = 16 rows of the ragged batch (dense numbering), y = layer; 256 threads
template <int kMode>
__global__ __launch_bounds__(256) void hash_score_kernel(
    const short* __restrict__ q_sum, const unsigned* __restrict__ qbar_codes,
    const short* __restrict__ colsum, int64_t cs_layer_stride, const unsigned* __restrict__ block_codes,
    int64_t bc_layer_stride, const int32_t* __restrict__ seg_off, const int32_t* __restrict__ seg_len,
    unsigned n_req, unsigned kv_heads, float* __restrict__ scores, int64_t scores_layer_stride, int round_fp16)
{
    const unsigned l = blockIdx.y;
    const unsigned sub = threadIdx.x & 15;
    int dense = blockIdx.x * 16 + (threadIdx.x >> 4);
    int r = -1, local = 0;
    for (unsigned i = 0; i < n_req; ++i) {
        const int n = max(seg_len[i], 0);
        if (dense < n) { r = static_cast<int>(i); local = dense; break; }
        dense -= n;
    }
    int score = 0;
    int64_t row = 0;
    if (r >= 0) {
        row = static_cast<int64_t>(seg_off[r]) + local;
        const size_t lr = static_cast<size_t>(l) * n_req + r;
        if (kMode == 0) {
            // <sum_i u(q_i), sum_h S[h]>
            const short* cs = colsum + static_cast<int64_t>(l) * cs_layer_stride + row * kv_heads * kBits + sub * 8;
            const i16x8 qv = *reinterpret_cast<const i16x8*>(q_sum + lr * kBits + sub * 8);
            int s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (unsigned h = 0; h < kv_heads; ++h) {
                const i16x8 v = *reinterpret_cast<const i16x8*>(cs + h * kBits);
#pragma unroll
                for (int k = 0; k < 8; ++k) { s[k] += v[k]; }
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) { score += static_cast<int>(qv[k]) * s[k]; }
        } else {
            // sum over kv heads of (bits - hamming(code of the group-mean query, majority code of the block))
            const unsigned* bc = block_codes + static_cast<int64_t>(l) * bc_layer_stride + row * kv_heads * 4;
            const unsigned* qc = qbar_codes + lr * kv_heads * 4;
            for (unsigned wd = sub; wd < kv_heads * 4; wd += 16) { score += 32 - __popc(bc[wd] ^ qc[wd]); }
        }
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

}  // namespace

extern "C" int ucm_hash_encode_blocks(const void* const* k_layers, int n_layers, int num_blocks,
                                      const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                      int kv_heads, int head_dim, const void* w_bf16, int bits, int rows,
                                      uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                                      int64_t colsum_layer_stride, uint8_t* block_codes,
                                      int64_t block_codes_layer_stride, ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0, "ucm_hash_encode_blocks: n=%d", n);
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
    hipLaunchKernelGGL(hash_encode_blocks_kernel, dim3((n + kWaves - 1) / kWaves, n_layers), dim3(kThreads), 0,
                       ucm::as_stream(stream), k_layers, block_ids, slots, static_cast<unsigned>(num_blocks),
                       static_cast<unsigned>(n), static_cast<unsigned>(rows), static_cast<unsigned>(block_size),
                       static_cast<unsigned>(kv_heads), static_cast<const unsigned short*>(w_bf16),
                       reinterpret_cast<unsigned*>(token_codes), token_codes_layer_stride / 4, colsum,
                       colsum_layer_stride, reinterpret_cast<unsigned*>(block_codes), block_codes_layer_stride / 4);
    UCM_LAUNCH_CHECK("ucm_hash_encode_blocks");
}

extern "C" int ucm_hash_encode_queries(const void* q_bf16, int64_t q_layer_stride, const int32_t* q_rows,
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
    UCM_SUPPORTED(q_heads <= kMaxQHeads, "ucm_hash_encode_queries: q_heads=%d (at most %d)", q_heads, kMaxQHeads);
    hipLaunchKernelGGL(hash_query_kernel, dim3(n_req, n_layers), dim3(kQueryThreads), 0, ucm::as_stream(stream),
                       static_cast<const unsigned short*>(q_bf16), q_layer_stride, q_rows,
                       static_cast<unsigned>(q_heads), static_cast<unsigned>(kv_heads),
                       static_cast<const unsigned short*>(w_bf16), static_cast<unsigned>(n_req),
                       reinterpret_cast<unsigned*>(q_codes), q_sum, reinterpret_cast<unsigned*>(qbar_codes));
    UCM_LAUNCH_CHECK("ucm_hash_encode_queries");
}

extern "C" int ucm_hash_score_blocks(int mode, const int16_t* q_sum, const uint8_t* qbar_codes,
                                     const int16_t* colsum, int64_t colsum_layer_stride,
                                     const uint8_t* block_codes, int64_t block_codes_layer_stride,
                                     const int32_t* seg_off, const int32_t* seg_len, int n_req,
                                     int64_t total_blocks, int n_layers, int kv_heads, int bits, float* scores,
                                     int64_t scores_layer_stride, int round_fp16, ucm_stream_t stream)
{
    UCM_REQUIRE(n_req >= 0 && total_blocks >= 0 && n_layers > 0 && n_layers <= 65535,
                "ucm_hash_score_blocks: n_req=%d n_layers=%d", n_req, n_layers);
    if (n_req == 0 || total_blocks == 0) { return UCM_OK; }
    UCM_REQUIRE(mode == 0 || mode == 1, "ucm_hash_score_blocks: mode=%d", mode);
    UCM_REQUIRE(seg_off && seg_len && scores, "ucm_hash_score_blocks: null pointer");
    UCM_REQUIRE(mode == 0 ? (q_sum && colsum) : (qbar_codes && block_codes), "ucm_hash_score_blocks: null operand for this mode");
    UCM_SUPPORTED(bits == kBits && kv_heads >= 1 && kv_heads <= kMaxHeads, "ucm_hash_score_blocks: bits=%d kv_heads=%d", bits, kv_heads);
    const unsigned gx = static_cast<unsigned>((total_blocks + 15) / 16);
    hipStream_t s = ucm::as_stream(stream);
    if (mode == 0) {
        hipLaunchKernelGGL(hash_score_kernel<0>, dim3(gx, n_layers), dim3(256), 0, s, q_sum,
                           reinterpret_cast<const unsigned*>(qbar_codes), colsum, colsum_layer_stride,
                           reinterpret_cast<const unsigned*>(block_codes), block_codes_layer_stride / 4, seg_off, seg_len,
                           static_cast<unsigned>(n_req), static_cast<unsigned>(kv_heads), scores, scores_layer_stride,
                           round_fp16);
    } else {
        hipLaunchKernelGGL(hash_score_kernel<1>, dim3(gx, n_layers), dim3(256), 0, s, q_sum,
                           reinterpret_cast<const unsigned*>(qbar_codes), colsum, colsum_layer_stride,
                           reinterpret_cast<const unsigned*>(block_codes), block_codes_layer_stride / 4, seg_off, seg_len,
                           static_cast<unsigned>(n_req), static_cast<unsigned>(kv_heads), scores, scores_layer_stride,
                           round_fp16);
    }
    UCM_LAUNCH_CHECK("ucm_hash_score_blocks");
}
