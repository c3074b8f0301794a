/*
 * Host twins of the C ABI: the same prototypes as libucm_hip.so's entry points
 * of the dense retrieval path, of the ESA retrieval worker, of the hash-code path, of the planned loads, of KVStar's
 * representatives, votes and selection and of the prefetch bookkeeping, name + "_cpu", every "dev" pointer a host
 * pointer, `stream` ignored, the work done before the call returns.  A caller
 * written against one prototype switches between host and device by choosing
 * the symbol.
 *
 * TEST INFRASTRUCTURE ONLY, like the rest of this directory: the arithmetic is
 * the oracle's (ucm_oracle.c, which names the reference lines it follows) and
 * nothing here is linked into, loaded by or shipped with the product.  The
 * twins are compiled into liborc.so.
 *
 * The type of every twin is taken from the device entry point's declaration
 * (`__typeof__`), so a twin whose parameter list drifts from the header does
 * not compile.  Argument checks follow the device library's: UCM_EINVAL for
 * what it calls a bad argument, ids / slots / rows outside their table are
 * skipped, never dereferenced.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "ucm_hip.h"

#define ORC_API __attribute__((visibility("default")))
#define TWIN(name) ORC_API extern __typeof__(name) name##_cpu

TWIN(ucm_block_mean);
TWIN(ucm_score_blocks);
TWIN(ucm_topk_windows);
TWIN(ucm_score_select);
TWIN(ucm_kv_gather_blocks);
TWIN(ucm_kv_scatter_blocks);
TWIN(ucm_kv_gather_blocks_tp);
TWIN(ucm_kv_scatter_blocks_tp);
TWIN(ucm_kv_load_planned_tp);
TWIN(ucm_kv_gather_selected);
TWIN(ucm_delta_plan);
TWIN(ucm_delta_plan_rows);
TWIN(ucm_esa_retrieve);
TWIN(ucm_esa_retrieve_rows);
TWIN(ucm_hash_encode_blocks);
TWIN(ucm_hash_encode_queries);
TWIN(ucm_hash_encode_blocks_f16);
TWIN(ucm_hash_encode_queries_f16);
TWIN(ucm_hash_score_blocks);
TWIN(ucm_copy_batch);
TWIN(ucm_kv_load_planned);
TWIN(ucm_kvstar_topk);
TWIN(ucm_kvstar_order);
TWIN(ucm_prefetch_plan);
TWIN(ucm_kvstar_block_repre);
TWIN(ucm_kvstar_block_repre_keys);
TWIN(ucm_kvstar_votes);
TWIN(ucm_kvstar_votes_tables);
TWIN(ucm_kvstar_park_queries);
TWIN(ucm_park_rows);

/* the oracle's functions these forward to (ucm_oracle.c) */
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);
void orc_block_mean_paged_f16(const uint16_t* k_cache, const int32_t* block_ids, const int32_t* slots, uint32_t n,
                              uint32_t blockSize, uint32_t kHead, uint32_t headSize, float* repre, int round_f16);
void orc_block_mean_paged(const uint16_t* k_cache, const int32_t* block_ids, const int32_t* slots, uint32_t n,
                          uint32_t blockSize, uint32_t kHead, uint32_t headSize, float* repre, int round_bf16);
void orc_q_head_mean(float* q, uint32_t kHead, uint32_t qHead, uint32_t headSize);
void orc_kq_scores(const float* qMean, const float* kRepre, uint32_t numBlock, uint32_t kHead, uint32_t numKrepre,
                   uint32_t headSize, float* scores);
int32_t orc_topk_windows(const float* scores, uint32_t n, uint32_t k, uint32_t startW, uint32_t endW, int32_t* out);
int32_t orc_block_table_gather(const int32_t* block_table, const int32_t* topk_idx, int32_t count, int32_t seq_len,
                               int32_t block_size, int32_t* phys_out);
int32_t orc_esa_retrieve(const float* data, uint32_t dim, const float* q, const int32_t* indexes, uint32_t n_indexes,
                         int32_t topk, int32_t* out_idx, float* out_scores);
int32_t orc_delta_plan(const int32_t* sel, const int32_t* sel_phys, int32_t count, int32_t* resident, int32_t n_slots,
                       int32_t* load_phys, int32_t* slot_of_sel);
void orc_hash_encode(const uint16_t* x, const float* W, uint32_t n, uint32_t dim, uint32_t bits, uint8_t* codes);
void orc_hash_encode_f32(const float* x, const float* W, uint32_t n, uint32_t dim, uint32_t bits, uint8_t* codes);
void orc_hash_colsum(const uint8_t* token_codes, uint32_t n_blocks, uint32_t block_size, uint32_t kv_heads, uint32_t nbytes,
                     int16_t* out);
void orc_hash_majority(const uint8_t* token_codes, uint32_t n_blocks, uint32_t block_size, uint32_t kv_heads, uint32_t nbytes,
                       uint8_t* block_codes);
void orc_hash_scores_block(const uint8_t* q_codes, const uint8_t* block_codes, uint32_t n_blocks, uint32_t kv_heads,
                           uint32_t nbytes, int32_t* scores);
float orc_f16_to_f32(uint16_t h);
int32_t orc_kvstar_topk(const float* final_scores, uint32_t n_blocks, uint32_t topk, int32_t* topk_idx);
void orc_kvstar_block_repre(const uint16_t* cache, const int32_t* block_ids, const int32_t* slots, uint32_t n, uint32_t block_size,
                            uint32_t kv_heads, uint32_t head_dim, uint32_t merge, const int32_t* pruned, uint32_t d_pruned,
                            uint32_t d_pad, uint16_t* repre);
void orc_kvstar_block_repre_f16(const uint16_t* cache, const int32_t* block_ids, const int32_t* slots, uint32_t n, uint32_t block_size,
                            uint32_t kv_heads, uint32_t head_dim, uint32_t merge, const int32_t* pruned, uint32_t d_pruned,
                            uint32_t d_pad, uint16_t* repre);
int32_t orc_kvstar_retrieve(const uint16_t* q, uint32_t n_tokens, uint32_t q_heads, uint32_t d_orig, const uint16_t* repre,
                            uint32_t n_blocks, uint32_t M, uint32_t kv_heads, uint32_t d_pruned, uint32_t d_pad,
                            const int32_t* pruned, uint32_t topk, float* final_scores, int32_t* topk_idx);
int32_t orc_prefetch_run(int32_t* map_block, int32_t* map_idx, int32_t n_map, const int32_t* topk, int32_t topk_len,
                         int32_t* free_block, int32_t* free_len, int32_t* success_blocks, int32_t success_cap,
                         int32_t* success_len, int32_t* load_blocks, int32_t* miss_idxs, int32_t* n_miss);
uint16_t orc_f32_to_f16(float f);

int ucm_block_mean_cpu(const void* const* k_layers, int n_layers, int num_blocks, const int32_t* block_ids,
                       const int32_t* slots, int n, int block_size, int kv_heads, int head_dim, void* repre,
                       int repre_rows, int64_t repre_layer_stride, int mode, ucm_stream_t stream)
{
    (void)stream;
    if (n < 0 || n_layers < 0) { return UCM_EINVAL; }
    if (n == 0 || n_layers == 0) { return UCM_OK; }
    if (!k_layers || !block_ids || !slots || !repre || num_blocks <= 0 || repre_rows <= 0 || block_size <= 0 ||
        kv_heads <= 0 || head_dim <= 0 || (mode & ~(UCM_MEAN_ABS | UCM_MEAN_KEYS_F16)) < UCM_MEAN_F32 ||
        (mode & ~(UCM_MEAN_ABS | UCM_MEAN_KEYS_F16)) > UCM_MEAN_BF16_STORE) {
        return UCM_EINVAL;
    }
    const int of_abs = (mode & UCM_MEAN_ABS) != 0, keys_f16 = (mode & UCM_MEAN_KEYS_F16) != 0;
    mode &= ~(UCM_MEAN_ABS | UCM_MEAN_KEYS_F16);
    if (keys_f16 && mode == UCM_MEAN_BF16_STORE) { return UCM_ENOTSUP; }
    void (*mean)(const uint16_t*, const int32_t*, const int32_t*, uint32_t, uint32_t, uint32_t, uint32_t, float*, int) =
        keys_f16 ? orc_block_mean_paged_f16 : orc_block_mean_paged;
    const size_t row = (size_t)kv_heads * head_dim;
    float* tmp = (float*)malloc(row * sizeof(float));
    uint16_t* blk = of_abs ? (uint16_t*)malloc((size_t)block_size * row * sizeof(uint16_t)) : NULL;   /* the block without its signs */
    if (!tmp || (of_abs && !blk)) { free(tmp); free(blk); return UCM_ENOMEM; }
    const int32_t zero = 0;
    for (int l = 0; l < n_layers; ++l) {
        for (int i = 0; i < n; ++i) {
            if (block_ids[i] < 0 || block_ids[i] >= num_blocks || slots[i] < 0 || slots[i] >= repre_rows) { continue; }
            if (of_abs) {
                const uint16_t* src = (const uint16_t*)k_layers[l] + (size_t)block_ids[i] * block_size * row;
                for (size_t e = 0; e < (size_t)block_size * row; ++e) { blk[e] = src[e] & 0x7fffu; }
                mean(blk, &zero, &zero, 1, (uint32_t)block_size, (uint32_t)kv_heads, (uint32_t)head_dim, tmp, mode != UCM_MEAN_F32);
            } else {
                mean((const uint16_t*)k_layers[l], &block_ids[i], &zero, 1, (uint32_t)block_size, (uint32_t)kv_heads,
                     (uint32_t)head_dim, tmp, mode != UCM_MEAN_F32);
            }
            const size_t at = (size_t)l * (size_t)repre_layer_stride + (size_t)slots[i] * row;
            if (mode == UCM_MEAN_BF16_STORE) {
                for (size_t c = 0; c < row; ++c) { ((uint16_t*)repre)[at + c] = orc_f32_to_bf16(tmp[c]); }
            } else {
                memcpy((float*)repre + at, tmp, row * sizeof(float));
            }
        }
    }
    free(tmp);
    free(blk);
    return UCM_OK;
}

static float widen_q(const void* q, int q_dtype, size_t at)
{
    if (q_dtype == UCM_DTYPE_F32) { return ((const float*)q)[at]; }
    return q_dtype == UCM_DTYPE_BF16 ? orc_bf16_to_f32(((const uint16_t*)q)[at]) : orc_f16_to_f32(((const uint16_t*)q)[at]);
}

/* scores of the requests whose descriptors may be followed (the device library's rule: query row inside the
 * layer's query block, rows inside [0, repre_rows)); the others are left alone */
static int score_host(const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows, int q_heads, const void* repre,
                      int repre_dtype, int64_t repre_layer_stride, int64_t repre_rows, int num_repre, const int32_t* seg_off,
                      const int32_t* seg_len, int n_req, int max_seg_len, int n_layers, int kv_heads, int head_dim, float* scores,
                      int64_t scores_layer_stride, float scale)
{
    if (n_req < 0 || max_seg_len < 0 || n_layers < 0 || !isfinite(scale) || repre_rows < 0 || num_repre < 1) { return UCM_EINVAL; }
    if (n_req == 0 || max_seg_len == 0 || n_layers == 0) { return UCM_OK; }
    if (!q || !repre || !seg_off || !seg_len || !scores || kv_heads <= 0 || q_heads < kv_heads ||
        q_heads % kv_heads != 0 || head_dim <= 0 || q_dtype < UCM_DTYPE_F32 || q_dtype > UCM_DTYPE_F16 ||
        (repre_dtype != UCM_DTYPE_F32 && repre_dtype != UCM_DTYPE_BF16)) {
        return UCM_EINVAL;
    }
    const size_t qrow = (size_t)q_heads * head_dim, row = (size_t)kv_heads * num_repre * head_dim;
    float* qf = (float*)malloc(qrow * sizeof(float));
    float* wide = (float*)malloc((size_t)max_seg_len * row * sizeof(float));
    if (!qf || !wide) { free(qf); free(wide); return UCM_ENOMEM; }
    for (int l = 0; l < n_layers; ++l) {
        for (int r = 0; r < n_req; ++r) {
            const int64_t qr = q_rows ? q_rows[r] : r;
            const int32_t n = seg_len[r] < max_seg_len ? seg_len[r] : max_seg_len;
            /* with q_rows, a layer's rows end at q_layer_stride: a request whose row lies outside is skipped */
            if (n <= 0 || qr < 0 || (q_rows && (int64_t)(qr + 1) * (int64_t)qrow > q_layer_stride)) { continue; }
            if (seg_off[r] < 0 || (int64_t)seg_off[r] + n > repre_rows) { continue; }
            const size_t q_at = (size_t)l * (size_t)q_layer_stride + (size_t)qr * qrow;
            for (size_t c = 0; c < qrow; ++c) { qf[c] = widen_q(q, q_dtype, q_at + c); }
            orc_q_head_mean(qf, (uint32_t)kv_heads, (uint32_t)q_heads, (uint32_t)head_dim);
            const size_t t_at = (size_t)l * (size_t)repre_layer_stride + (size_t)seg_off[r] * row;
            const float* table;
            if (repre_dtype == UCM_DTYPE_F32) {
                table = (const float*)repre + t_at;
            } else {
                for (size_t c = 0; c < (size_t)n * row; ++c) { wide[c] = orc_bf16_to_f32(((const uint16_t*)repre)[t_at + c]); }
                table = wide;
            }
            float* out = scores + (size_t)l * (size_t)scores_layer_stride + seg_off[r];
            orc_kq_scores(qf, table, (uint32_t)n, (uint32_t)kv_heads, (uint32_t)num_repre, (uint32_t)head_dim, out);
            for (int32_t b = 0; b < n; ++b) { out[b] = out[b] * scale; }
        }
    }
    free(qf);
    free(wide);
    return UCM_OK;
}

int ucm_score_blocks_cpu(const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows, int q_heads,
                         const void* repre, int repre_dtype, int64_t repre_layer_stride, int64_t repre_rows, int num_repre,
                         const int32_t* seg_off, const int32_t* seg_len, int n_req, int max_seg_len, int64_t total_blocks,
                         int n_layers, int kv_heads, int head_dim, float* scores, int64_t scores_layer_stride, float scale,
                         int tile_blocks, ucm_stream_t stream)
{
    (void)stream;
    (void)total_blocks;
    (void)tile_blocks;
    return score_host(q, q_dtype, q_layer_stride, q_rows, q_heads, repre, repre_dtype, repre_layer_stride, repre_rows, num_repre,
                      seg_off, seg_len, n_req, max_seg_len, n_layers, kv_heads, head_dim, scores, scores_layer_stride, scale);
}

int ucm_topk_windows_cpu(const float* scores, int64_t scores_layer_stride, int64_t scores_rows, const int32_t* seg_off,
                         const int32_t* seg_len, const int32_t* topk_len, int n_req, int max_seg_len, int n_layers, int start_w,
                         int end_w, int32_t* idx_out, int out_stride, int32_t* count_out, const int32_t* block_tables,
                         int bt_stride, int32_t* phys_out, const int32_t* seq_lens, int block_size, int32_t* sparse_seq_lens,
                         ucm_stream_t stream)
{
    (void)stream;
    if (n_req < 0 || n_layers < 0 || max_seg_len < 0 || start_w < 0 || end_w < 0 || scores_rows < 0) { return UCM_EINVAL; }
    if (n_req == 0 || n_layers == 0) { return UCM_OK; }
    if (!scores || !seg_off || !seg_len || !topk_len || !idx_out || !count_out || out_stride < max_seg_len ||
        (block_tables && (!phys_out || bt_stride < max_seg_len)) || (seq_lens && (!sparse_seq_lens || block_size <= 0))) {
        return UCM_EINVAL;
    }
    for (int l = 0; l < n_layers; ++l) {
        for (int r = 0; r < n_req; ++r) {
            const size_t lr = (size_t)l * n_req + r;
            int32_t n = seg_len[r] < max_seg_len ? seg_len[r] : max_seg_len;
            /* a request whose scores do not lie inside the layer selects nothing */
            if (n > 0 && (seg_off[r] < 0 || (int64_t)seg_off[r] + n > scores_rows)) { n = 0; }
            int32_t* out = idx_out + lr * (size_t)out_stride;
            int32_t cnt = 0;
            if (n > 0) {
                cnt = orc_topk_windows(scores + (size_t)l * (size_t)scores_layer_stride + seg_off[r], (uint32_t)n,
                                       (uint32_t)(topk_len[r] > 0 ? topk_len[r] : 0), (uint32_t)start_w, (uint32_t)end_w, out);
            }
            count_out[lr] = cnt;
            int32_t sparse = 0;
            if (block_tables) {
                sparse = orc_block_table_gather(block_tables + (size_t)r * bt_stride, out, cnt, seq_lens ? seq_lens[r] : 0,
                                                block_size > 0 ? block_size : 1, phys_out + lr * (size_t)out_stride);
            }
            if (seq_lens) {
                if (!block_tables) {
                    const int32_t rem = seq_lens[r] % block_size;
                    sparse = rem == 0 ? cnt * block_size : cnt * block_size - block_size + rem;
                }
                /* every block kept: the request is not sparsified and keeps its length (prefetch_engine.py:547-553) */
                sparse_seq_lens[lr] = cnt >= n ? seq_lens[r] : sparse;
            }
        }
    }
    return UCM_OK;
}

/* the one-launch entry point: scores, then the selection from them, on layers first_layer .. */
int ucm_score_select_cpu(const ucm_score_select_args_t* p, ucm_stream_t stream)
{
    if (!p || p->struct_size != sizeof(ucm_score_select_args_t) || p->n_req < 0 || p->n_layers <= 0 || p->first_layer < 0) {
        return UCM_EINVAL;
    }
    if (p->n_req == 0) { return UCM_OK; }
    if (!p->tickets || !p->scores || p->max_seg_len < 0) { return UCM_EINVAL; }
    if (p->max_seg_len > 1024) { return UCM_ENOTSUP; }
    const int64_t es = p->repre_dtype == UCM_DTYPE_BF16 ? 2 : 4;
    const int first = p->first_layer;
    const char* repre = (const char*)p->repre + (int64_t)first * p->repre_layer_stride * es;
    float* scores = p->scores + (int64_t)first * p->scores_layer_stride;
    const int64_t idx_ls = p->idx_layer_stride ? p->idx_layer_stride : (int64_t)p->n_req * p->out_stride;
    const int64_t cnt_ls = p->count_layer_stride ? p->count_layer_stride : p->n_req;
    if (idx_ls < (int64_t)p->n_req * p->out_stride || cnt_ls < p->n_req) { return UCM_EINVAL; }
    int rc = score_host(p->q, p->q_dtype, p->q_layer_stride, p->q_rows, p->q_heads, repre, p->repre_dtype, p->repre_layer_stride,
                        p->repre_rows, p->num_repre, p->seg_off, p->seg_len, p->n_req, p->max_seg_len, p->n_layers, p->kv_heads,
                        p->head_dim, scores, p->scores_layer_stride, p->scale);
    /* the selection layer by layer: the tables' layers may lie further apart than a dense layer */
    for (int l = 0; l < p->n_layers && rc == UCM_OK; ++l) {
        const int64_t li = (first + l) * idx_ls, lc = (first + l) * cnt_ls;
        rc = ucm_topk_windows_cpu(scores + (int64_t)l * p->scores_layer_stride, p->scores_layer_stride, p->repre_rows, p->seg_off,
                                  p->seg_len, p->topk_len, p->n_req, p->max_seg_len, 1, p->start_w, p->end_w, p->idx_out + li,
                                  p->out_stride, p->count_out + lc, p->block_tables, p->bt_stride,
                                  p->phys_out ? p->phys_out + li : NULL, p->seq_lens, p->block_size,
                                  p->sparse_seq_lens ? p->sparse_seq_lens + lc : NULL, stream);
    }
    return rc;
}

int64_t orc_get_offset(int64_t block_size, int64_t kv_heads_per_tp, int64_t head_size, int64_t rank, int64_t tp_size,
                       int64_t precision, int64_t layer_id, int is_v, int is_mla);

/* where get_offset puts a rank's K or V slice of a layer inside a stored block (a slice is block_bytes long) */
static size_t stored_slice(size_t block_bytes, int rank, int tp_size, int layer, int kv)
{
    return (size_t)orc_get_offset((int64_t)block_bytes, 1, 1, rank, tp_size, 1, layer, kv, 0);
}

static int kv_move(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                   const int32_t* block_ids, int n, void* staging, int to_staging, int rank, int tp_size)
{
    if (n < 0 || n_layers < 0 || tp_size < 1 || rank < 0 || rank >= tp_size) { return UCM_EINVAL; }
    if (n == 0 || n_layers == 0) { return UCM_OK; }
    if (!layers || !block_ids || !staging || num_blocks <= 0 || block_bytes == 0) { return UCM_EINVAL; }
    for (int i = 0; i < n; ++i) {
        if (block_ids[i] < 0 || block_ids[i] >= num_blocks) { continue; }
        for (int l = 0; l < n_layers; ++l) {
            for (int kv = 0; kv < 2; ++kv) {
                uint8_t* c = (uint8_t*)layers[l] + (size_t)kv * kv_stride + (size_t)block_ids[i] * block_bytes;
                uint8_t* s = (uint8_t*)staging + (size_t)i * n_layers * 2 * block_bytes * tp_size +
                             stored_slice(block_bytes, rank, tp_size, l, kv);
                if (to_staging) { memcpy(s, c, block_bytes); } else { memcpy(c, s, block_bytes); }
            }
        }
    }
    return UCM_OK;
}

int ucm_kv_gather_blocks_cpu(const void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                             const int32_t* block_ids, int n, void* staging, ucm_stream_t stream)
{
    (void)stream;
    return kv_move((void* const*)layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, staging, 1, 0, 1);
}

int ucm_kv_gather_blocks_tp_cpu(const void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                                const int32_t* block_ids, int n, void* staging, int rank, int tp_size, ucm_stream_t stream)
{
    (void)stream;
    return kv_move((void* const*)layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, staging, 1, rank, tp_size);
}

int ucm_kv_scatter_blocks_cpu(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                              const int32_t* block_ids, int n, const void* staging, ucm_stream_t stream)
{
    (void)stream;
    return kv_move(layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, (void*)staging, 0, 0, 1);
}

int ucm_kv_scatter_blocks_tp_cpu(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                                 const int32_t* block_ids, int n, const void* staging, int rank, int tp_size,
                                 ucm_stream_t stream)
{
    (void)stream;
    return kv_move(layers, n_layers, kv_stride, block_bytes, num_blocks, block_ids, n, (void*)staging, 0, rank, tp_size);
}

int ucm_kv_gather_selected_cpu(const void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                               const int32_t* phys, const int32_t* count, int n_req, int phys_stride, const int64_t* dst_off,
                               const int32_t* region_k, int max_count, void* staging, int64_t staging_blocks,
                               ucm_stream_t stream)
{
    (void)stream;
    if (n_req < 0 || n_layers < 0 || max_count < 0) { return UCM_EINVAL; }
    if (n_req == 0 || n_layers == 0 || max_count == 0) { return UCM_OK; }
    if (!layers || !phys || !count || !dst_off || !region_k || !staging || num_blocks <= 0 || block_bytes == 0 ||
        phys_stride <= 0 || staging_blocks < 0) {
        return UCM_EINVAL;
    }
    for (int l = 0; l < n_layers; ++l) {
        for (int r = 0; r < n_req; ++r) {
            int32_t c = count[(size_t)l * n_req + r];
            if (c > max_count) { c = max_count; }
            if (dst_off[r] < 0 || region_k[r] < 0) { continue; }
            for (int kv = 0; kv < 2; ++kv) {
                for (int32_t j = 0; j < c; ++j) {
                    const int32_t id = phys[((size_t)l * n_req + r) * (size_t)phys_stride + j];
                    const int64_t dst = dst_off[r] + ((int64_t)l * 2 + kv) * region_k[r] + j;
                    /* an id outside the cache (-1 marks a slot a delta plan leaves alone) or a destination
                     * outside the staging buffer is skipped */
                    if (id < 0 || id >= num_blocks || dst >= staging_blocks) { continue; }
                    memcpy((uint8_t*)staging + (size_t)dst * block_bytes,
                           (const uint8_t*)layers[l] + (size_t)kv * kv_stride + (size_t)id * block_bytes, block_bytes);
                }
            }
        }
    }
    return UCM_OK;
}

int ucm_delta_plan_cpu(const int32_t* sel, const int32_t* sel_phys, const int32_t* count, int n_req, int n_layers,
                       int sel_stride, int32_t* resident, int n_slots, int32_t* load_phys, int32_t* slot_of_sel,
                       int32_t* miss_count, ucm_stream_t stream)
{
    (void)stream;
    if (n_req < 0 || n_layers < 0) { return UCM_EINVAL; }
    if (n_req == 0 || n_layers == 0) { return UCM_OK; }
    if (!sel || !sel_phys || !count || !resident || !load_phys || !slot_of_sel || !miss_count || sel_stride <= 0 ||
        n_slots <= 0) {
        return UCM_EINVAL;
    }
    for (size_t lr = 0; lr < (size_t)n_layers * n_req; ++lr) {
        int32_t c = count[lr] < 0 ? 0 : count[lr];
        if (c > sel_stride) { c = sel_stride; }
        miss_count[lr] = orc_delta_plan(sel + lr * (size_t)sel_stride, sel_phys + lr * (size_t)sel_stride, c,
                                        resident + lr * (size_t)n_slots, n_slots, load_phys + lr * (size_t)n_slots,
                                        slot_of_sel + lr * (size_t)sel_stride);
    }
    return UCM_OK;
}

int ucm_delta_plan_rows_cpu(const int32_t* sel, const int32_t* sel_phys, const int32_t* count, const int32_t* rows, int batch,
                            int table_rows, int n_layers, int sel_stride, int32_t* resident, int n_slots, int32_t* load_phys,
                            int32_t* slot_of_sel, int32_t* miss_count, ucm_stream_t stream)
{
    (void)stream;
    if (batch < 0 || table_rows <= 0 || n_layers <= 0) { return UCM_EINVAL; }
    if (batch == 0) { return UCM_OK; }
    if (!sel || !sel_phys || !count || !rows || !resident || !load_phys || !slot_of_sel || !miss_count || sel_stride < 1) {
        return UCM_EINVAL;
    }
    if (n_slots < 1 || n_slots > 1024) { return UCM_ENOTSUP; }
    for (int l = 0; l < n_layers; ++l) {
        for (int b = 0; b < batch; ++b) {
            if (rows[b] < 0 || rows[b] >= table_rows) { continue; }
            const size_t lr = (size_t)l * table_rows + rows[b];
            int32_t c = count[lr] < 0 ? 0 : count[lr];
            if (c > sel_stride) { c = sel_stride; }
            miss_count[lr] = orc_delta_plan(sel + lr * (size_t)sel_stride, sel_phys + lr * (size_t)sel_stride, c,
                                            resident + lr * (size_t)n_slots, n_slots, load_phys + lr * (size_t)n_slots,
                                            slot_of_sel + lr * (size_t)sel_stride);
        }
    }
    return UCM_OK;
}

/* ------------------------------------------------------- ESA retrieval */

/*
 * One request: the list entries that name a row of the table go to orc_esa_retrieve in list order (it breaks ties by
 * that order); a winner's position in the list is the first position not yet given out that holds its row.
 */
static int esa_one(const float* data, int n_items, int dim, const float* q, const int32_t* list, int m, int topk,
                   int32_t* out_idx, int32_t* out_pos, float* out_scores)
{
    int32_t* keep = (int32_t*)malloc(((size_t)m + 1) * sizeof(int32_t));
    int32_t* pos = (int32_t*)malloc(((size_t)m + 1) * sizeof(int32_t));
    int32_t* win = (int32_t*)malloc(((size_t)m + 1) * sizeof(int32_t));
    float* win_s = (float*)malloc(((size_t)m + 1) * sizeof(float));
    char* used = (char*)calloc((size_t)m + 1, 1);
    int n = 0, got = -1;
    if (keep && pos && win && win_s && used) {
        for (int j = 0; j < m; ++j) {
            if (list[j] >= 0 && list[j] < n_items) { keep[n] = list[j]; pos[n] = j; ++n; }
        }
        got = orc_esa_retrieve(data, (uint32_t)dim, q, keep, (uint32_t)n, topk, win, win_s);
        for (int i = 0; i < got; ++i) {
            int at = 0;
            while (used[at] || keep[at] != win[i]) { ++at; }
            used[at] = 1;
            out_idx[i] = win[i];
            out_scores[i] = win_s[i];
            if (out_pos) { out_pos[i] = pos[at]; }
        }
    }
    free(keep); free(pos); free(win); free(win_s); free(used);
    return got;
}

static int esa_check(const float* data, int n_items, int dim, const float* q, const void* lists, int batch, int m, int topk,
                     const void* ws, const void* out_idx, const void* out_scores, const void* out_count, int out_stride)
{
    if (batch < 0 || m < 0) { return UCM_EINVAL; }
    if (batch == 0) { return 1; }                        /* nothing to do */
    if (!data || !q || !out_idx || !out_scores || !out_count || (m > 0 && (!lists || !ws)) || n_items <= 0 || dim <= 0) {
        return UCM_EINVAL;
    }
    if (dim % 4 != 0) { return UCM_ENOTSUP; }
    const int k = topk < 0 ? 0 : topk;
    if (batch > 65535 || out_stride < (k < m ? k : m)) { return UCM_EINVAL; }
    return m > 8192 ? UCM_ENOTSUP : UCM_OK;
}

int ucm_esa_retrieve_cpu(const float* data, int n_items, int dim, const float* q, const int32_t* indexes, int batch, int m,
                         int topk, float* scores_ws, int32_t* out_idx, float* out_scores, int32_t* out_count, int out_stride,
                         ucm_stream_t stream)
{
    (void)stream;
    const int rc = esa_check(data, n_items, dim, q, indexes, batch, m, topk, scores_ws, out_idx, out_scores, out_count, out_stride);
    if (rc != UCM_OK) { return rc == 1 ? UCM_OK : rc; }
    for (int b = 0; b < batch; ++b) {
        const int got = esa_one(data, n_items, dim, q + (size_t)b * dim, indexes + (size_t)b * m, m, topk,
                                out_idx + (size_t)b * out_stride, NULL, out_scores + (size_t)b * out_stride);
        if (got < 0) { return UCM_ENOMEM; }
        out_count[b] = got;
    }
    return UCM_OK;
}

int ucm_esa_retrieve_rows_cpu(const float* data, int n_items, int dim, const float* q, const int32_t* slot_table,
                              int table_rows, int table_stride, int m, const int32_t* rows, int batch, const int32_t* topk_rows,
                              int max_topk, float* scores_ws, int32_t* out_idx, int32_t* out_pos, float* out_scores,
                              int32_t* out_count, int out_stride, ucm_stream_t stream)
{
    (void)stream;
    const int rc = esa_check(data, n_items, dim, q, slot_table, batch, m, max_topk, scores_ws, out_idx, out_scores, out_count,
                             out_stride);
    if (rc != UCM_OK) { return rc == 1 ? UCM_OK : rc; }
    if (!rows || !topk_rows || table_rows <= 0 || table_stride < m) { return UCM_EINVAL; }
    for (int b = 0; b < batch; ++b) {
        const int row = rows[b];
        if (row < 0 || row >= table_rows) { continue; }
        const int k = topk_rows[row] < max_topk ? topk_rows[row] : max_topk;
        const int got = esa_one(data, n_items, dim, q + (size_t)b * dim, slot_table + (size_t)row * table_stride, m, k,
                                out_idx + (size_t)row * out_stride, out_pos ? out_pos + (size_t)row * out_stride : NULL,
                                out_scores + (size_t)row * out_stride);
        if (got < 0) { return UCM_ENOMEM; }
        out_count[row] = got;
    }
    return UCM_OK;
}

/* ------------------------------------------------------------ hash codes */

/* bfloat16 or float16 values widened to fp32 (exact either way) */
static void widen_to_f32(const void* src, int f16, size_t n, float* dst)
{
    for (size_t i = 0; i < n; ++i) {
        const uint16_t h = ((const uint16_t*)src)[i];
        dst[i] = f16 ? orc_f16_to_f32(h) : orc_bf16_to_f32(h);
    }
}

static float* widen_weights(const void* w16, int f16, int head_dim, int bits)
{
    float* w = (float*)malloc((size_t)head_dim * bits * sizeof(float));
    if (w) { widen_to_f32(w16, f16, (size_t)head_dim * bits, w); }
    return w;
}

static int hash_encode_blocks_host(int f16, const void* const* k_layers, int n_layers, int num_blocks, const int32_t* block_ids,
                                   const int32_t* slots, int n, int block_size, int kv_heads, int head_dim, const void* w_bf16,
                                   int bits, int rows, uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                                   int64_t colsum_layer_stride, uint8_t* block_codes, int64_t block_codes_layer_stride)
{
    if (n < 0) { return UCM_EINVAL; }
    if (n == 0) { return UCM_OK; }
    if (!k_layers || !w_bf16 || !colsum || !block_codes || n_layers <= 0 || num_blocks <= 0 || rows <= 0 || block_size <= 0 ||
        kv_heads <= 0) {
        return UCM_EINVAL;
    }
    if (head_dim != 128 || bits != 128) { return UCM_ENOTSUP; }
    const uint32_t nbytes = (uint32_t)bits / 8;
    const size_t n_vec = (size_t)block_size * kv_heads;
    float* w = widen_weights(w_bf16, f16, head_dim, bits);
    uint8_t* codes = (uint8_t*)malloc(n_vec * nbytes);
    float* xf = f16 ? (float*)malloc(n_vec * head_dim * sizeof(float)) : NULL;
    if (!w || !codes || (f16 && !xf)) { free(w); free(codes); free(xf); return UCM_ENOMEM; }
    for (int l = 0; l < n_layers; ++l) {
        for (int i = 0; i < n; ++i) {
            /* block_ids NULL: item i is block i; slots NULL: it goes to row i */
            const int64_t id = block_ids ? block_ids[i] : i, slot = slots ? slots[i] : i;
            if (id < 0 || id >= num_blocks || slot < 0 || slot >= rows) { continue; }
            const uint16_t* x = (const uint16_t*)k_layers[l] + (size_t)id * n_vec * head_dim;
            if (f16) {
                widen_to_f32(x, 1, n_vec * head_dim, xf);
                orc_hash_encode_f32(xf, w, (uint32_t)n_vec, (uint32_t)head_dim, (uint32_t)bits, codes);
            } else {
                orc_hash_encode(x, w, (uint32_t)n_vec, (uint32_t)head_dim, (uint32_t)bits, codes);
            }
            if (token_codes) {
                memcpy(token_codes + (size_t)l * (size_t)token_codes_layer_stride + (size_t)slot * n_vec * nbytes, codes,
                       n_vec * nbytes);
            }
            orc_hash_colsum(codes, 1, (uint32_t)block_size, (uint32_t)kv_heads, nbytes,
                            colsum + (size_t)l * (size_t)colsum_layer_stride + (size_t)slot * kv_heads * bits);
            orc_hash_majority(codes, 1, (uint32_t)block_size, (uint32_t)kv_heads, nbytes,
                              block_codes + (size_t)l * (size_t)block_codes_layer_stride + (size_t)slot * kv_heads * nbytes);
        }
    }
    free(w);
    free(codes);
    free(xf);
    return UCM_OK;
}

int ucm_hash_encode_blocks_cpu(const void* const* k_layers, int n_layers, int num_blocks, const int32_t* block_ids,
                               const int32_t* slots, int n, int block_size, int kv_heads, int head_dim, const void* w_bf16,
                               int bits, int rows, uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                               int64_t colsum_layer_stride, uint8_t* block_codes, int64_t block_codes_layer_stride,
                               int workgroups, ucm_stream_t stream)
{
    (void)stream;
    (void)workgroups;
    return hash_encode_blocks_host(0, k_layers, n_layers, num_blocks, block_ids, slots, n, block_size, kv_heads, head_dim, w_bf16,
                                   bits, rows, token_codes, token_codes_layer_stride, colsum, colsum_layer_stride, block_codes,
                                   block_codes_layer_stride);
}

int ucm_hash_encode_blocks_f16_cpu(const void* const* k_layers, int n_layers, int num_blocks, const int32_t* block_ids,
                                   const int32_t* slots, int n, int block_size, int kv_heads, int head_dim, const void* w_f16,
                                   int bits, int rows, uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                                   int64_t colsum_layer_stride, uint8_t* block_codes, int64_t block_codes_layer_stride,
                                   int workgroups, ucm_stream_t stream)
{
    (void)stream;
    (void)workgroups;
    return hash_encode_blocks_host(1, k_layers, n_layers, num_blocks, block_ids, slots, n, block_size, kv_heads, head_dim, w_f16,
                                   bits, rows, token_codes, token_codes_layer_stride, colsum, colsum_layer_stride, block_codes,
                                   block_codes_layer_stride);
}

static int hash_encode_queries_host(int f16, const void* q_bf16, int64_t q_layer_stride, const int32_t* q_rows, int n_req,
                                    int n_layers, int q_heads, int kv_heads, int head_dim, const void* w_bf16, int bits,
                                    uint8_t* q_codes, int16_t* q_sum, uint8_t* qbar_codes)
{
    if (n_req < 0 || n_layers < 0) { return UCM_EINVAL; }
    if (n_req == 0 || n_layers == 0) { return UCM_OK; }
    if (!q_bf16 || !w_bf16 || !q_codes || !q_sum || !qbar_codes || kv_heads <= 0 || q_heads < kv_heads ||
        q_heads % kv_heads != 0) {
        return UCM_EINVAL;
    }
    if (head_dim != 128 || bits != 128) { return UCM_ENOTSUP; }
    const uint32_t nbytes = (uint32_t)bits / 8;
    const size_t qrow = (size_t)q_heads * head_dim;
    float* w = widen_weights(w_bf16, f16, head_dim, bits);
    float* qf = (float*)malloc(qrow * sizeof(float));
    if (!w || !qf) { free(w); free(qf); return UCM_ENOMEM; }
    for (int l = 0; l < n_layers; ++l) {
        for (int r = 0; r < n_req; ++r) {
            const int64_t qr = q_rows ? q_rows[r] : r;
            if (qr < 0 || (q_rows && (int64_t)(qr + 1) * (int64_t)qrow > q_layer_stride)) { continue; }   /* left as they were */
            const uint16_t* x = (const uint16_t*)q_bf16 + (size_t)l * (size_t)q_layer_stride + (size_t)qr * qrow;
            const size_t lr = (size_t)l * n_req + r;
            uint8_t* codes = q_codes + lr * q_heads * nbytes;
            widen_to_f32(x, f16, qrow, qf);
            orc_hash_encode_f32(qf, w, (uint32_t)q_heads, (uint32_t)head_dim, (uint32_t)bits, codes);
            for (int c = 0; c < bits; ++c) {
                int32_t ones = 0;
                for (int h = 0; h < q_heads; ++h) { ones += (codes[(size_t)h * nbytes + c / 8] >> (c % 8)) & 1; }
                q_sum[lr * bits + c] = (int16_t)(2 * ones - q_heads);
            }
            /* the kv head's group-mean query in fp32 (select_topk_block.cpp:101-114), then its code */
            orc_q_head_mean(qf, (uint32_t)kv_heads, (uint32_t)q_heads, (uint32_t)head_dim);
            orc_hash_encode_f32(qf, w, (uint32_t)kv_heads, (uint32_t)head_dim, (uint32_t)bits, qbar_codes + lr * kv_heads * nbytes);
        }
    }
    free(w);
    free(qf);
    return UCM_OK;
}

int ucm_hash_encode_queries_cpu(const void* q_bf16, int64_t q_layer_stride, const int32_t* q_rows, int n_req, int n_layers,
                                int q_heads, int kv_heads, int head_dim, const void* w_bf16, int bits, uint8_t* q_codes,
                                int16_t* q_sum, uint8_t* qbar_codes, ucm_stream_t stream)
{
    (void)stream;
    return hash_encode_queries_host(0, q_bf16, q_layer_stride, q_rows, n_req, n_layers, q_heads, kv_heads, head_dim, w_bf16, bits,
                                    q_codes, q_sum, qbar_codes);
}

int ucm_hash_encode_queries_f16_cpu(const void* q_f16, int64_t q_layer_stride, const int32_t* q_rows, int n_req, int n_layers,
                                    int q_heads, int kv_heads, int head_dim, const void* w_f16, int bits, uint8_t* q_codes,
                                    int16_t* q_sum, uint8_t* qbar_codes, ucm_stream_t stream)
{
    (void)stream;
    return hash_encode_queries_host(1, q_f16, q_layer_stride, q_rows, n_req, n_layers, q_heads, kv_heads, head_dim, w_f16, bits,
                                    q_codes, q_sum, qbar_codes);
}

int ucm_hash_score_blocks_cpu(int mode, const int16_t* q_sum, const uint8_t* qbar_codes, const int16_t* colsum,
                              int64_t colsum_layer_stride, const uint8_t* block_codes, int64_t block_codes_layer_stride,
                              int64_t rows, const int32_t* seg_off, const int32_t* seg_len, int n_req, int64_t total_blocks, int n_layers,
                              int kv_heads, int bits, float* scores, int64_t scores_layer_stride, int round_fp16,
                              ucm_stream_t stream)
{
    (void)stream;
    (void)total_blocks;
    if (n_req < 0 || n_layers < 0 || (mode != 0 && mode != 1) || rows < 0) { return UCM_EINVAL; }
    if (n_req == 0 || n_layers == 0) { return UCM_OK; }
    if (!seg_off || !seg_len || !scores || kv_heads <= 0 || (mode == 0 && (!q_sum || !colsum)) ||
        (mode == 1 && (!qbar_codes || !block_codes))) {
        return UCM_EINVAL;
    }
    if (bits != 128) { return UCM_ENOTSUP; }
    const uint32_t nbytes = (uint32_t)bits / 8;
    for (int l = 0; l < n_layers; ++l) {
        for (int r = 0; r < n_req; ++r) {
            const size_t lr = (size_t)l * n_req + r;
            /* a request whose rows do not lie inside the summary tables is not scored */
            if (seg_off[r] < 0 || (int64_t)seg_off[r] + (seg_len[r] > 0 ? seg_len[r] : 0) > rows) { continue; }
            float* out = scores + (size_t)l * (size_t)scores_layer_stride + seg_off[r];
            for (int32_t b = 0; b < seg_len[r]; ++b) {
                const size_t row = (size_t)seg_off[r] + b;
                if (mode == 0) {
                    /* <sum of the query heads' +-1 codes, sum over kv heads of the block's column sums>: the reference's
                     * triple sum of +-1 inner products (kvcomp.py:237-247) as one integer */
                    int64_t s = 0;
                    const int16_t* cs = colsum + (size_t)l * (size_t)colsum_layer_stride + row * kv_heads * bits;
                    for (int c = 0; c < bits; ++c) {
                        int32_t col = 0;
                        for (int h = 0; h < kv_heads; ++h) { col += cs[(size_t)h * bits + c]; }
                        s += (int64_t)q_sum[lr * bits + c] * col;
                    }
                    float f = (float)s;
                    out[b] = round_fp16 ? orc_f16_to_f32(orc_f32_to_f16(f)) : f;
                } else {
                    int32_t s = 0;
                    orc_hash_scores_block(qbar_codes + lr * kv_heads * nbytes,
                                          block_codes + (size_t)l * (size_t)block_codes_layer_stride + row * kv_heads * nbytes, 1,
                                          (uint32_t)kv_heads, nbytes, &s);
                    out[b] = (float)s;
                }
            }
        }
    }
    return UCM_OK;
}

/* ---- pointer-array copy and planned loads ------------------------------------------------------------------ */

int ucm_copy_batch_cpu(void* const* dst, const void* const* src, size_t num, size_t size, ucm_stream_t stream)
{
    (void)stream;
    if (num == 0 || size == 0) { return UCM_OK; }
    if (!dst || !src || size % 16) { return UCM_EINVAL; }
    for (size_t i = 0; i < num; ++i) {
        if (!dst[i] || !src[i] || ((uintptr_t)dst[i] | (uintptr_t)src[i]) % 16) { return UCM_EINVAL; }
    }
    for (size_t i = 0; i < num; ++i) { memmove(dst[i], src[i], size); }
    return UCM_OK;
}

int ucm_park_rows_cpu(const void* src, int64_t src_rows, const int32_t* src_idx, void* dst, int64_t dst_rows,
                      const int32_t* dst_idx, int n, size_t row_bytes, ucm_stream_t stream)
{
    (void)stream;
    if (n < 0 || src_rows < 0 || dst_rows < 0 || row_bytes == 0 || row_bytes % 16) { return UCM_EINVAL; }
    if (n == 0) { return UCM_OK; }
    if (!src || !src_idx || !dst || ((uintptr_t)src | (uintptr_t)dst) % 16) { return UCM_EINVAL; }
    for (int i = 0; i < n; ++i) {
        const int64_t from = src_idx[i], to = dst_idx ? dst_idx[i] : i;
        if (from < 0 || from >= src_rows || to < 0 || to >= dst_rows) { continue; }
        memmove((char*)dst + (size_t)to * row_bytes, (const char*)src + (size_t)from * row_bytes, row_bytes);
    }
    return UCM_OK;
}

int ucm_kv_load_planned_tp_cpu(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                               const void* pool, int64_t pool_blocks, size_t pool_block_bytes, int store_first_layer,
                               const int32_t* load_sel, int n_slots, const int32_t* src_table, int src_stride,
                               const int32_t* dst_table, int dst_stride, int64_t dst_layer_stride, const int32_t* load_count,
                               const int32_t* rows, int batch, int table_rows, int rank, int tp_size, ucm_stream_t stream)
{
    (void)stream;
    if (batch < 0 || n_slots < 0 || table_rows <= 0 || tp_size < 1 || rank < 0 || rank >= tp_size) { return UCM_EINVAL; }
    if (batch == 0 || n_slots == 0) { return UCM_OK; }
    if (!layers || !pool || !load_sel || !src_table || !dst_table || n_layers <= 0 || num_blocks <= 0 || block_bytes == 0 ||
        block_bytes % 16 || kv_stride % 16 || pool_block_bytes % 16 || (size_t)num_blocks * block_bytes > kv_stride ||
        store_first_layer < 0 || pool_blocks < 0 || src_stride < 1 || dst_stride < n_slots || dst_layer_stride < 0 ||
        (size_t)(store_first_layer + n_layers) * 2 * block_bytes * tp_size > pool_block_bytes) {
        return UCM_EINVAL;
    }
    for (int l = 0; l < n_layers; ++l) {
        for (int b = 0; b < batch; ++b) {
            const int row = rows ? rows[b] : b;
            if (row < 0 || row >= table_rows) { continue; }
            int limit = n_slots;
            if (load_count) {
                const int32_t c = load_count[(size_t)l * table_rows + row];
                if (c < limit) { limit = c < 0 ? 0 : c; }
            }
            for (int j = 0; j < limit; ++j) {
                const int32_t sel = load_sel[((size_t)l * table_rows + row) * (size_t)n_slots + j];
                if (sel < 0 || sel >= src_stride) { continue; }
                const int32_t from = src_table[(size_t)row * src_stride + sel];
                if (from < 0 || from >= pool_blocks) { continue; }
                const int32_t to = dst_table[l * dst_layer_stride + (int64_t)row * dst_stride + j];
                if (to < 0 || to >= num_blocks) { continue; }
                for (int kv = 0; kv < 2; ++kv) {
                    memcpy((uint8_t*)layers[l] + (size_t)kv * kv_stride + (size_t)to * block_bytes,
                           (const uint8_t*)pool + (size_t)from * pool_block_bytes +
                               stored_slice(block_bytes, rank, tp_size, store_first_layer + l, kv),
                           block_bytes);
                }
            }
        }
    }
    return UCM_OK;
}

int ucm_kv_load_planned_cpu(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes, int num_blocks,
                            const void* pool, int64_t pool_blocks, size_t pool_block_bytes, int store_first_layer,
                            const int32_t* load_sel, int n_slots, const int32_t* src_table, int src_stride,
                            const int32_t* dst_table, int dst_stride, int64_t dst_layer_stride, const int32_t* load_count,
                            const int32_t* rows, int batch, int table_rows, ucm_stream_t stream)
{
    return ucm_kv_load_planned_tp_cpu(layers, n_layers, kv_stride, block_bytes, num_blocks, pool, pool_blocks, pool_block_bytes,
                                      store_first_layer, load_sel, n_slots, src_table, src_stride, dst_table, dst_stride,
                                      dst_layer_stride, load_count, rows, batch, table_rows, 0, 1, stream);
}

/* ---- KVStar's selection ----------------------------------------------------------------------------------------- */

static int cmp_i32(const void* a, const void* b)
{
    const int32_t x = *(const int32_t*)a, y = *(const int32_t*)b;
    return (x > y) - (x < y);
}

int ucm_kvstar_topk_cpu(const float* votes, int64_t votes_rows, const int32_t* seg_off, const int32_t* seg_len,
                        const int32_t* topk_len, int n_tasks, int max_seg_len, int32_t* idx_out, int out_stride,
                        int32_t* count_out, ucm_stream_t stream)
{
    (void)stream;
    if (n_tasks < 0 || max_seg_len < 0 || votes_rows < 0) { return UCM_EINVAL; }
    if (n_tasks == 0) { return UCM_OK; }
    if (!votes || !seg_off || !seg_len || !topk_len || !idx_out || !count_out || out_stride < max_seg_len) { return UCM_EINVAL; }
    if (max_seg_len > 4096) { return UCM_ENOTSUP; }
    for (int t = 0; t < n_tasks; ++t) {
        int n = seg_len[t] < max_seg_len ? seg_len[t] : max_seg_len;
        if (n > out_stride) { n = out_stride; }
        if (n > 0 && (seg_off[t] < 0 || (int64_t)seg_off[t] + n > votes_rows)) { n = 0; }   /* votes outside the array */
        int32_t* out = idx_out + (size_t)t * out_stride;
        if (n <= 0) { count_out[t] = 0; continue; }
        const int32_t k = topk_len[t];
        int32_t got;
        if (k <= 0 || k >= n) {                      /* everything, as ucm_topk_windows hands it out */
            for (int i = 0; i < n; ++i) { out[i] = i; }
            got = n;
        } else {
            got = orc_kvstar_topk(votes + seg_off[t], (uint32_t)n, (uint32_t)k, out);   /* the heap's order */
            qsort(out, (size_t)got, sizeof(int32_t), cmp_i32);                          /* the device's: ascending */
        }
        count_out[t] = got;
    }
    return UCM_OK;
}

int ucm_kvstar_order_cpu(const float* votes, int64_t votes_rows, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                         int max_count, int32_t* idx_io, int out_stride, const int32_t* count, ucm_stream_t stream)
{
    (void)stream;
    if (n_tasks < 0 || max_count < 0 || votes_rows < 0) { return UCM_EINVAL; }
    if (n_tasks == 0 || max_count == 0) { return UCM_OK; }
    if (!votes || !seg_off || !seg_len || !idx_io || !count || out_stride < max_count) { return UCM_EINVAL; }
    if (max_count > 4096) { return UCM_ENOTSUP; }
    for (int t = 0; t < n_tasks; ++t) {
        int32_t* row = idx_io + (size_t)t * out_stride;
        int k = count[t];
        if (k > out_stride) { k = out_stride; }
        if (k > 4096) { k = 4096; }
        if (seg_off[t] < 0 || seg_len[t] < 0 || (int64_t)seg_off[t] + seg_len[t] > votes_rows) { continue; }
        const float* v = votes + seg_off[t];
        /* descending by (vote, index): insertion sort, the lists are short; the two zeros compare equal */
        for (int a = 1; a < k; ++a) {
            const int32_t cur = row[a];
            int b = a - 1;
            while (b >= 0 && (v[row[b]] < v[cur] || (v[row[b]] == v[cur] && row[b] < cur))) {
                row[b + 1] = row[b];
                --b;
            }
            row[b + 1] = cur;
        }
    }
    return UCM_OK;
}

/* ---- GSA prefetch bookkeeping ------------------------------------------------------------------------------------ */

int ucm_prefetch_plan_cpu(const int32_t* map_block, const int32_t* map_len, int32_t* map_idx, int table_rows, int cap,
                          const int32_t* topk_idx, int topk_stride, const int32_t* topk_len, const int32_t* rows,
                          const int32_t* bs_index, int batch, int n_layers, int max_bs, int row_len, int32_t* free_block,
                          int32_t* free_len, int32_t* success_blocks, int32_t* success_len, int32_t* load_blocks,
                          int32_t* load_count, int32_t* miss_idxs, int32_t* miss_count, ucm_stream_t stream)
{
    (void)stream;
    if (batch < 0 || n_layers <= 0) { return UCM_EINVAL; }
    if (batch == 0) { return UCM_OK; }
    if (!map_block || !map_len || !map_idx || !topk_idx || !topk_len || !rows || !bs_index || !free_block || !free_len ||
        !success_blocks || !success_len || !load_blocks || !load_count || !miss_idxs || !miss_count || table_rows <= 0 ||
        max_bs <= 0) {
        return UCM_EINVAL;
    }
    if (cap < 1 || cap > 256 || topk_stride < 1 || topk_stride > 256 || row_len < 1) { return UCM_ENOTSUP; }
    int32_t* blocks = (int32_t*)malloc(sizeof(int32_t) * 256 * 6);
    if (!blocks) { return UCM_ENOMEM; }
    int32_t* loads = blocks + 256;
    int32_t* misses = blocks + 512;
    int32_t* free_tmp = blocks + 768;
    int32_t* succ_tmp = blocks + 1024;                  /* 512 entries: hits and served misses */
    int rc = UCM_OK;
    for (int l = 0; l < n_layers && rc == UCM_OK; ++l) {
        for (int i = 0; i < batch; ++i) {
            const int row = rows[i], b = bs_index[i];
            int k = topk_len[i] < topk_stride ? topk_len[i] : topk_stride;
            if (row < 0 || row >= table_rows || b < 0 || b >= max_bs || k <= 0) {   /* the reference skips such a request */
                if (row >= 0 && row < table_rows) {
                    load_count[(size_t)l * table_rows + row] = 0;
                    miss_count[(size_t)l * table_rows + row] = 0;
                }
                continue;
            }
            const size_t lb = (size_t)l * max_bs + b, lr = (size_t)l * table_rows + row;
            int n = map_len[row] < cap ? map_len[row] : cap;
            if (n < 0) { n = 0; }
            int32_t f = free_len[lb] < row_len ? free_len[lb] : row_len;
            if (f > 256) { f = 256; }
            if (f < 0) { f = 0; }
            memcpy(blocks, map_block + (size_t)row * cap, sizeof(int32_t) * (size_t)n);
            memcpy(free_tmp, free_block + lb * row_len, sizeof(int32_t) * (size_t)f);
            int32_t n_succ = 0, n_miss = 0;
            const int32_t n_load = orc_prefetch_run(blocks, map_idx + lr * cap, n, topk_idx + ((size_t)l * batch + i) * topk_stride,
                                                    k, free_tmp, &f, succ_tmp, 512, &n_succ, loads, misses, &n_miss);
            if (n_load < 0) { rc = UCM_EINVAL; break; }      /* a free-list entry that is no block of the map */
            memcpy(load_blocks + lr * cap, loads, sizeof(int32_t) * (size_t)n_load);
            memcpy(miss_idxs + lr * topk_stride, misses, sizeof(int32_t) * (size_t)n_miss);
            for (int p = 0; p < row_len; ++p) { success_blocks[lb * row_len + p] = p < 512 ? succ_tmp[p] : 0; }
            memcpy(free_block + lb * row_len, free_tmp, sizeof(int32_t) * (size_t)(f < row_len ? f : row_len));
            free_len[lb] = f;
            success_len[lb] = n_succ;
            load_count[lr] = n_load;
            miss_count[lr] = n_miss;
        }
    }
    free(blocks);
    return rc;
}

/* ---- KVStar's representatives and votes ------------------------------------------------------------------------
 * The device keeps a block's sub-block representatives as cells [d_pad/8][M][8] per (layer, kv head, row) - the
 * order the score kernel streams; the oracle's functions use the reference's [row][M][kv head][d].  The twins move
 * between the two around the oracle's arithmetic.  The votes are the oracle's scalar loop: the device's agree with
 * them to rounding (other summation order on the matrix cores), not bit for bit. */

int ucm_kvstar_block_repre_cpu(const void* const* k_layers, int n_layers, int num_blocks, const int32_t* block_ids,
                               const int32_t* slots, int n, int block_size, int kv_heads, int head_dim, int merge,
                               const int32_t* pruned, int64_t pruned_layer_stride, const int32_t* pruned_sel, int n_pruned_lists,
                               int d_pruned, int d_pad, void* repre_f16, int repre_rows, int64_t repre_layer_stride,
                               int64_t repre_head_stride, int64_t repre_row_stride, ucm_stream_t stream)
{
    return ucm_kvstar_block_repre_keys_cpu(k_layers, UCM_DTYPE_BF16, n_layers, num_blocks, block_ids, slots, n, block_size, kv_heads,
                                           head_dim, merge, pruned, pruned_layer_stride, pruned_sel, n_pruned_lists, d_pruned, d_pad,
                                           repre_f16, repre_rows, repre_layer_stride, repre_head_stride, repre_row_stride, stream);
}

int ucm_kvstar_block_repre_keys_cpu(const void* const* k_layers, int key_dtype, int n_layers, int num_blocks,
                                    const int32_t* block_ids, const int32_t* slots, int n, int block_size, int kv_heads,
                                    int head_dim, int merge, const int32_t* pruned, int64_t pruned_layer_stride,
                                    const int32_t* pruned_sel, int n_pruned_lists, int d_pruned, int d_pad, void* repre_f16,
                                    int repre_rows, int64_t repre_layer_stride, int64_t repre_head_stride,
                                    int64_t repre_row_stride, ucm_stream_t stream)
{
    (void)stream;
    if (key_dtype != UCM_DTYPE_BF16 && key_dtype != UCM_DTYPE_F16) { return UCM_EINVAL; }
    if (n < 0 || n_layers < 0 || (pruned_sel && (!pruned || n_pruned_lists < 1))) { return UCM_EINVAL; }
    if (n == 0 || n_layers == 0) { return UCM_OK; }
    if (!k_layers || !repre_f16 || num_blocks <= 0 || repre_rows <= 0 || block_size <= 0 || kv_heads <= 0 || head_dim <= 0 ||
        merge <= 0 || block_size % merge || d_pruned <= 0 || d_pruned > head_dim || d_pad < d_pruned || d_pad % 8 ||
        (!pruned && d_pruned != head_dim) || (pruned_layer_stride != 0 && pruned_layer_stride < (int64_t)kv_heads * d_pruned) ||
        (repre_layer_stride | repre_head_stride | repre_row_stride) % 8) {
        return UCM_EINVAL;
    }
    const int M = block_size / merge;
    uint16_t* tmp = (uint16_t*)malloc((size_t)M * kv_heads * d_pad * sizeof(uint16_t));
    if (!tmp) { return UCM_ENOMEM; }
    const int32_t zero = 0;
    for (int l = 0; l < n_layers; ++l) {
        const int32_t* lists = pruned ? pruned + (int64_t)l * pruned_layer_stride : NULL;
        for (int i = 0; i < n; ++i) {
            const int32_t id = block_ids ? block_ids[i] : i, slot = slots ? slots[i] : i;
            if (id < 0 || id >= num_blocks || slot < 0 || slot >= repre_rows) { continue; }
            if (pruned_sel && (pruned_sel[i] < 0 || pruned_sel[i] >= n_pruned_lists)) { continue; }   /* a list that does not exist */
            const int32_t* mine = (lists && pruned_sel) ? lists + (size_t)pruned_sel[i] * kv_heads * d_pruned : lists;
            (key_dtype == UCM_DTYPE_F16 ? orc_kvstar_block_repre_f16 : orc_kvstar_block_repre)(
                (const uint16_t*)k_layers[l], &id, &zero, 1, (uint32_t)block_size, (uint32_t)kv_heads, (uint32_t)head_dim,
                (uint32_t)merge, mine, (uint32_t)d_pruned, (uint32_t)d_pad, tmp);
            for (int h = 0; h < kv_heads; ++h) {
                uint16_t* cell = (uint16_t*)repre_f16 + (int64_t)l * repre_layer_stride + (int64_t)h * repre_head_stride +
                                 (int64_t)slot * repre_row_stride;
                for (int m = 0; m < M; ++m) {
                    for (int p = 0; p < d_pad; ++p) {
                        cell[((size_t)(p / 8) * M + m) * 8 + p % 8] = tmp[((size_t)m * kv_heads + h) * d_pad + p];
                    }
                }
            }
        }
    }
    free(tmp);
    return UCM_OK;
}

int ucm_kvstar_park_queries_cpu(const void* q, int q_dtype, int64_t q_rows, int row_elems, const int32_t* src_rows,
                                const int64_t* dst_off, int n, void* ring_f16, int64_t ring_elems, ucm_stream_t stream)
{
    (void)stream;
    if (n < 0 || q_rows < 0 || ring_elems < 0) { return UCM_EINVAL; }
    if (n == 0) { return UCM_OK; }
    if (!q || !src_rows || !dst_off || !ring_f16 || q_dtype < UCM_DTYPE_F32 || q_dtype > UCM_DTYPE_F16 || row_elems <= 0 ||
        row_elems % 8) {
        return UCM_EINVAL;
    }
    for (int i = 0; i < n; ++i) {
        const int64_t src = src_rows[i], dst = dst_off[i];
        if (src < 0 || src >= q_rows || dst < 0 || dst + row_elems > ring_elems || (dst & 7)) { continue; }
        for (int e = 0; e < row_elems; ++e) {
            const size_t at = (size_t)src * row_elems + e;
            uint16_t h;
            if (q_dtype == UCM_DTYPE_F16) { h = ((const uint16_t*)q)[at]; }
            else if (q_dtype == UCM_DTYPE_BF16) { h = orc_f32_to_f16(orc_bf16_to_f32(((const uint16_t*)q)[at])); }
            else { h = orc_f32_to_f16(((const float*)q)[at]); }
            ((uint16_t*)ring_f16)[dst + e] = h;
        }
    }
    return UCM_OK;
}

/* votes of one task whose block b has its cell of kv head h at table + h*head_stride + b*row_stride */
static int kvstar_task_votes(const uint16_t* q, int n_tokens, int q_heads, int d_orig, const int32_t* lists, const uint16_t* table,
                             int64_t head_stride, int64_t row_stride, int n_blocks, int M, int kv_heads, int d_pruned, int d_pad,
                             float* votes)
{
    if (n_blocks <= 0) { return UCM_OK; }
    uint16_t* ref = (uint16_t*)malloc((size_t)n_blocks * M * kv_heads * d_pad * sizeof(uint16_t));
    if (!ref) { return UCM_ENOMEM; }
    for (int b = 0; b < n_blocks; ++b) {
        for (int h = 0; h < kv_heads; ++h) {
            const uint16_t* cell = table + (int64_t)h * head_stride + (int64_t)b * row_stride;
            for (int m = 0; m < M; ++m) {
                for (int p = 0; p < d_pad; ++p) {
                    ref[(((size_t)b * M + m) * kv_heads + h) * d_pad + p] = cell[((size_t)(p / 8) * M + m) * 8 + p % 8];
                }
            }
        }
    }
    int32_t none;
    orc_kvstar_retrieve(q, (uint32_t)n_tokens, (uint32_t)q_heads, (uint32_t)d_orig, ref, (uint32_t)n_blocks, (uint32_t)M,
                        (uint32_t)kv_heads, (uint32_t)d_pruned, (uint32_t)d_pad, lists, 0, votes, &none);
    free(ref);
    return UCM_OK;
}

/* the device library's rule for a task's descriptors: query block inside the buffer, channel list inside the lists,
 * rows inside the table / the votes array; a task outside any of them is skipped */
static int kvstar_task_ok(int64_t q_elems, const int64_t* q_off, int64_t q_need, int n_lists, const int32_t* pruned_sel,
                          int64_t rows_bound, const int32_t* seg_off, int n, int t)
{
    return q_off[t] >= 0 && q_off[t] + q_need <= q_elems && (!pruned_sel || pruned_sel[t] < n_lists) && seg_off[t] >= 0 &&
           (int64_t)seg_off[t] + (n > 0 ? n : 0) <= rows_bound;
}

static int kvstar_votes_check(const void* q, const int64_t* q_off, int n_tokens, int q_heads, int d_orig, const int32_t* pruned,
                              const int32_t* pruned_sel, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                              int max_blocks, int sub_blocks, int kv_heads, int d_pruned, int d_pad, const float* votes)
{
    if (n_tasks < 0 || max_blocks < 0) { return UCM_EINVAL; }
    if (n_tasks == 0) { return UCM_OK; }
    if (!q || !q_off || !seg_off || !seg_len || !votes || n_tokens <= 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads ||
        d_orig <= 0 || d_pruned <= 0 || d_pruned > d_orig || d_pad < d_pruned || (pruned == NULL) != (pruned_sel == NULL) ||
        (!pruned && d_pruned != d_orig) || sub_blocks <= 0) {
        return UCM_EINVAL;
    }
    if (n_tokens * (q_heads / kv_heads) > 64 || kv_heads > 8 || d_pad % 16 || d_pad > 128 || sub_blocks > 128 ||
        (sub_blocks & (sub_blocks - 1))) {
        return UCM_ENOTSUP;
    }
    return 1;   /* go on */
}

int ucm_kvstar_votes_cpu(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads, int d_orig,
                         const int32_t* pruned, int n_pruned_lists, const int32_t* pruned_sel, const void* repre_f16,
                         int64_t repre_rows, int64_t repre_head_stride, int64_t repre_row_stride, const int32_t* seg_off,
                         const int32_t* seg_len, int n_tasks, int max_blocks, int sub_blocks, int kv_heads, int d_pruned,
                         int d_pad, float* ws_max, int64_t ws_max_floats, float* ws_part, int64_t ws_part_floats, float* votes,
                         int tiles_per_wave, ucm_stream_t stream)
{
    (void)ws_max; (void)ws_max_floats; (void)ws_part; (void)ws_part_floats; (void)tiles_per_wave; (void)stream;
    const int rc = kvstar_votes_check(q_f16, q_off, n_tokens, q_heads, d_orig, pruned, pruned_sel, seg_off, seg_len, n_tasks,
                                      max_blocks, sub_blocks, kv_heads, d_pruned, d_pad, votes);
    if (rc != 1) { return rc; }
    if (!repre_f16 || q_elems < 0 || repre_rows < 0 || n_pruned_lists < 0) { return UCM_EINVAL; }
    for (int t = 0; t < n_tasks; ++t) {
        const int n = seg_len[t] < max_blocks ? seg_len[t] : max_blocks;
        if (!kvstar_task_ok(q_elems, q_off, (int64_t)n_tokens * q_heads * d_orig, n_pruned_lists, pruned_sel, repre_rows, seg_off, n, t)) {
            continue;
        }
        const int32_t* lists = (pruned && pruned_sel[t] >= 0) ? pruned + (size_t)pruned_sel[t] * kv_heads * d_pruned : NULL;
        const int r = kvstar_task_votes((const uint16_t*)q_f16 + q_off[t], n_tokens, q_heads, d_orig, lists,
                                        (const uint16_t*)repre_f16 + (int64_t)seg_off[t] * repre_row_stride, repre_head_stride,
                                        repre_row_stride, n, sub_blocks, kv_heads, d_pruned, d_pad, votes + seg_off[t]);
        if (r != UCM_OK) { return r; }
    }
    return UCM_OK;
}

int ucm_kvstar_votes_tables_cpu(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads, int d_orig,
                                const int32_t* pruned, int n_pruned_lists, const int32_t* pruned_sel,
                                const void* const* task_tables, const int64_t* task_head_strides, int64_t task_row_stride,
                                const int32_t* seg_off, const int32_t* seg_len, int n_tasks, int max_blocks, int sub_blocks,
                                int kv_heads, int d_pruned, int d_pad, float* ws_max, int64_t ws_max_floats, float* ws_part,
                                int64_t ws_part_floats, float* votes, int64_t votes_rows, int tiles_per_wave, ucm_stream_t stream)
{
    (void)ws_max; (void)ws_max_floats; (void)ws_part; (void)ws_part_floats; (void)tiles_per_wave; (void)stream;
    const int rc = kvstar_votes_check(q_f16, q_off, n_tokens, q_heads, d_orig, pruned, pruned_sel, seg_off, seg_len, n_tasks,
                                      max_blocks, sub_blocks, kv_heads, d_pruned, d_pad, votes);
    if (rc != 1) { return rc; }
    if (!task_tables || !task_head_strides || q_elems < 0 || votes_rows < 0 || n_pruned_lists < 0) { return UCM_EINVAL; }
    for (int t = 0; t < n_tasks; ++t) {
        const int n = seg_len[t] < max_blocks ? seg_len[t] : max_blocks;
        if (!kvstar_task_ok(q_elems, q_off, (int64_t)n_tokens * q_heads * d_orig, n_pruned_lists, pruned_sel, votes_rows, seg_off, n, t)) {
            continue;
        }
        const int32_t* lists = (pruned && pruned_sel[t] >= 0) ? pruned + (size_t)pruned_sel[t] * kv_heads * d_pruned : NULL;
        const int r = kvstar_task_votes((const uint16_t*)q_f16 + q_off[t], n_tokens, q_heads, d_orig, lists,
                                        (const uint16_t*)task_tables[t], task_head_strides[t], task_row_stride, n, sub_blocks,
                                        kv_heads, d_pruned, d_pad, votes + seg_off[t]);
        if (r != UCM_OK) { return r; }
    }
    return UCM_OK;
}

