// Block representatives: per (kv head, dim) mean over a cache block's tokens,
// fp32 accumulation in token order (column-independent, so every thread owns
// whole columns and the order inside a column is the reference's).
//
// HBM-bound: block_size*row*2 bytes read per block, row*4 written.  A token
// row of the key cache ([kv_heads][head_dim] bf16, or fp16 for a model that runs in float16) is contiguous, so a thread
// owns 8 adjacent columns (one 16-byte load per token) and a workgroup of 128
// threads covers 1024 columns = one whole Llama-shape row; the token loop is
// unrolled 16 deep so 16 x 2 KiB of loads are in flight per workgroup.
#include "common.h"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 128;
constexpr int kCols = 8;      // bf16 columns per thread
constexpr int kUnroll = 16;   // token rows in flight

__device__ __forceinline__ float bf16_lo(unsigned w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }

__device__ __forceinline__ float round_bf16(float x)
{
    unsigned u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) { return __uint_as_float((u | 0x00400000u) & 0xffff0000u); }
    u += 0x7fffu + ((u >> 16) & 1u);
    return __uint_as_float(u & 0xffff0000u);
}

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// fp32 -> fp16 -> fp32, the fp32 value rounded once more.  The value is made opaque first: handed a product, the
// compiler otherwise folds the multiplication into a mixed-precision instruction that rounds the exact product
// straight to fp16 - one rounding instead of the two the reference's arithmetic has (seen at a tie: 1/5 of a sum).
__device__ __forceinline__ float round_f16(float x)
{
    asm volatile("" : "+v"(x));
    return static_cast<float>(static_cast<_Float16>(x));
}

// kAbs: the absolute values (a pair of 16-bit floats of either kind loses its two sign bits with one AND);
// kF16: the cache holds fp16 keys, not bf16 ones
template <bool kAbs, bool kF16>
__device__ __forceinline__ void widen(u32x4 v, float (&f)[kCols])
{
    if (kAbs) { v.x &= 0x7fff7fffu; v.y &= 0x7fff7fffu; v.z &= 0x7fff7fffu; v.w &= 0x7fff7fffu; }
    if (kF16) {
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f16x2 p = __builtin_bit_cast(f16x2, w[j]);
            f[2 * j] = static_cast<float>(p[0]);
            f[2 * j + 1] = static_cast<float>(p[1]);
        }
        return;
    }
    f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x);
    f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
    f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z);
    f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
}

// acc += token rows t .. t+kN-1, in that order, all kN loads issued before the first add
template <int kN, bool kAbs, bool kF16>
__device__ __forceinline__ void add_rows(const uint16_t* __restrict__ base, unsigned row, unsigned t, float (&acc)[kCols])
{
    u32x4 v[kN];
#pragma unroll
    for (int u = 0; u < kN; ++u) { v[u] = ucm::gload16_nt(base + static_cast<size_t>(t + u) * row); }
#pragma unroll
    for (int u = 0; u < kN; ++u) {
        float f[kCols];
        widen<kAbs, kF16>(v[u], f);
#pragma unroll
        for (int c = 0; c < kCols; ++c) { acc[c] = acc[c] + f[c]; }
    }
}

// grid: x = block index in the list * col_groups + column group of 1024, y = layer; rows narrower than 1024
// columns whose thread count divides the workgroup (a tensor-parallel rank's 4, 2 or 1 kv heads of 128) share a
// workgroup, items_per_group list entries side by side, so that no lane idles
template <bool kAbs, bool kF16>
__global__ __launch_bounds__(kThreads) void block_mean_kernel(
    const void* const* __restrict__ k_layers, const int32_t* __restrict__ block_ids,
    const int32_t* __restrict__ slots, unsigned num_blocks, unsigned repre_rows, unsigned block_size,
    unsigned row /* kv_heads*head_dim */, float* __restrict__ repre, int64_t repre_layer_stride,
    int round_to_bf16, unsigned col_groups, unsigned items_per_group, unsigned n_items)
{
    unsigned item, col;
    if (items_per_group > 1) {
        const unsigned per_item = kThreads / items_per_group;
        item = blockIdx.x * items_per_group + threadIdx.x / per_item;
        col = (threadIdx.x % per_item) * kCols;
        if (item >= n_items) { return; }
    } else {
        item = blockIdx.x / col_groups;
        col = ((blockIdx.x % col_groups) * kThreads + threadIdx.x) * kCols;
    }
    if (col >= row) { return; }
    const unsigned id = static_cast<unsigned>(block_ids[item]);
    const unsigned slot = static_cast<unsigned>(slots[item]);
    if (id >= num_blocks || slot >= repre_rows) { return; }  // never dereference a bad id

    const uint16_t* base = static_cast<const uint16_t*>(k_layers[blockIdx.y]) +
                           static_cast<size_t>(id) * block_size * row + col;
    float acc[kCols];
    widen<kAbs, kF16>(ucm::gload16(base), acc);  // acc = token 0

    unsigned t = 1;
    // full groups of kUnroll tokens: loads first, then the ordered adds; what is left (all of a 16-token block
    // after its first token) goes in groups of 8, 4, 2 and 1, each with its loads issued together
    for (; t + kUnroll <= block_size; t += kUnroll) { add_rows<kUnroll, kAbs, kF16>(base, row, t, acc); }
    if (t + 8 <= block_size) { add_rows<8, kAbs, kF16>(base, row, t, acc); t += 8; }
    if (t + 4 <= block_size) { add_rows<4, kAbs, kF16>(base, row, t, acc); t += 4; }
    if (t + 2 <= block_size) { add_rows<2, kAbs, kF16>(base, row, t, acc); t += 2; }
    if (t < block_size) { add_rows<1, kAbs, kF16>(base, row, t, acc); }

    const float inv = 1.0f / static_cast<float>(block_size);
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
        acc[c] = acc[c] * inv;
        if (round_to_bf16) { acc[c] = kF16 ? round_f16(acc[c]) : round_bf16(acc[c]); }
    }
    if (round_to_bf16 == 2) {
        // bf16 table: the rounded means themselves, 16 bytes per thread
        uint16_t* out16 = reinterpret_cast<uint16_t*>(repre) + static_cast<int64_t>(blockIdx.y) * repre_layer_stride +
                          static_cast<size_t>(slot) * row + col;
        u32x4 packed;
        packed.x = (__float_as_uint(acc[0]) >> 16) | (__float_as_uint(acc[1]) & 0xffff0000u);
        packed.y = (__float_as_uint(acc[2]) >> 16) | (__float_as_uint(acc[3]) & 0xffff0000u);
        packed.z = (__float_as_uint(acc[4]) >> 16) | (__float_as_uint(acc[5]) & 0xffff0000u);
        packed.w = (__float_as_uint(acc[6]) >> 16) | (__float_as_uint(acc[7]) & 0xffff0000u);
        *reinterpret_cast<u32x4*>(out16) = packed;
        return;
    }
    float* out = repre + static_cast<int64_t>(blockIdx.y) * repre_layer_stride +
                 static_cast<size_t>(slot) * row + col;
    f32x4 lo = {acc[0], acc[1], acc[2], acc[3]};
    f32x4 hi = {acc[4], acc[5], acc[6], acc[7]};
    *reinterpret_cast<f32x4*>(out) = lo;
    *reinterpret_cast<f32x4*>(out + 4) = hi;
}

}  // namespace

extern "C" int ucm_block_mean(const void* const* k_layers, int n_layers, int num_blocks,
                              const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                              int kv_heads, int head_dim, void* repre, int repre_rows,
                              int64_t repre_layer_stride, int mode, ucm_stream_t stream)
{
    UCM_REQUIRE(n >= 0, "ucm_block_mean: n=%d", n);
    if (n == 0) { return UCM_OK; }  // an empty list has no pointers to check
    UCM_REQUIRE(k_layers && block_ids && slots && repre, "ucm_block_mean: null pointer");
    UCM_REQUIRE(n_layers > 0 && n_layers <= 65535, "ucm_block_mean: n_layers=%d", n_layers);
    UCM_REQUIRE(block_size > 0 && kv_heads > 0 && head_dim > 0 && num_blocks > 0 && repre_rows > 0,
                "ucm_block_mean: non-positive shape");
    const bool of_abs = (mode & UCM_MEAN_ABS) != 0, keys_f16 = (mode & UCM_MEAN_KEYS_F16) != 0;
    mode &= ~(UCM_MEAN_ABS | UCM_MEAN_KEYS_F16);
    UCM_REQUIRE(mode == UCM_MEAN_F32 || mode == UCM_MEAN_BF16_ROUND || mode == UCM_MEAN_BF16_STORE,
                "ucm_block_mean: mode=%d", mode);
    UCM_SUPPORTED(!(keys_f16 && mode == UCM_MEAN_BF16_STORE), "ucm_block_mean: no bf16 table from an fp16 key cache "
                  "(UCM_MEAN_F32 or UCM_MEAN_BF16_ROUND, which then rounds to fp16)");
    const unsigned row = static_cast<unsigned>(kv_heads) * static_cast<unsigned>(head_dim);
    UCM_SUPPORTED(row % kCols == 0, "ucm_block_mean: kv_heads*head_dim=%u must be a multiple of %d", row, kCols);
    UCM_REQUIRE(repre_layer_stride >= static_cast<int64_t>(repre_rows) * row || n_layers == 1,
                "ucm_block_mean: repre_layer_stride=%lld smaller than one layer's table",
                static_cast<long long>(repre_layer_stride));
    UCM_REQUIRE(ucm::aligned16(repre) && (repre_layer_stride % (mode == UCM_MEAN_BF16_STORE ? 8 : 4) == 0),
                "ucm_block_mean: repre not 16-byte aligned");
    const unsigned gx = (row / kCols + kThreads - 1) / kThreads;
    UCM_REQUIRE(static_cast<uint64_t>(n) * gx <= 0x7fffffffull, "ucm_block_mean: too many blocks for one launch");
    const unsigned per_item = row / kCols;               // threads a list entry needs
    const unsigned share = (per_item < kThreads && kThreads % per_item == 0) ? kThreads / per_item : 1u;
    const unsigned groups = share > 1 ? (static_cast<unsigned>(n) + share - 1) / share : static_cast<unsigned>(n) * gx;
#define UCM_BLOCK_MEAN_ARGS dim3(groups, n_layers), dim3(kThreads), 0, ucm::as_stream(stream), k_layers, block_ids, slots, \
        static_cast<unsigned>(num_blocks), static_cast<unsigned>(repre_rows), static_cast<unsigned>(block_size), row,       \
        static_cast<float*>(repre), repre_layer_stride, mode, gx, share, static_cast<unsigned>(n)
    if (keys_f16) {
        if (of_abs) { hipLaunchKernelGGL((block_mean_kernel<true, true>), UCM_BLOCK_MEAN_ARGS); }
        else { hipLaunchKernelGGL((block_mean_kernel<false, true>), UCM_BLOCK_MEAN_ARGS); }
    } else if (of_abs) {
        hipLaunchKernelGGL((block_mean_kernel<true, false>), UCM_BLOCK_MEAN_ARGS);
    } else {
        hipLaunchKernelGGL((block_mean_kernel<false, false>), UCM_BLOCK_MEAN_ARGS);
    }
#undef UCM_BLOCK_MEAN_ARGS
    UCM_LAUNCH_CHECK("ucm_block_mean");
}
