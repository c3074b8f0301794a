/*
 * libucm_hip.so - C ABI of the MI355X (gfx950) sparse-retrieval hot path.
 *
 * Plain pointers and sizes only; every pointer marked "dev" is device memory
 * (anything a HIP kernel can dereference, which includes mapped pinned host
 * memory for the staging side of the KV moves).  The library allocates nothing
 * and never synchronises: each call validates its arguments on the host,
 * enqueues its kernels on `stream` (a hipStream_t, NULL = the null stream) and
 * returns.  Return value: 0 on success, a negative errno-style code otherwise
 * (UCM_EINVAL bad argument, UCM_ENOTSUP shape outside what the kernels were
 * built for, UCM_EHIP a HIP runtime error, UCM_ENOMEM an allocation that was
 * refused); ucm_last_error() has the text.
 *
 * Reference paths are relative to the upstream tree; each entry point names
 * the reference interface it stands in for.
 *
 * Shared conventions
 *   layers      dev array of n_layers pointers, one per model layer.  For the
 *               KV moves a layer pointer is the start of that layer's
 *               (2, num_blocks, block_size, kv_heads, head_dim) cache (K plane
 *               first, V plane kv_stride bytes later: vLLM layout,
 *               ucm/sparse/gsa/gsa.py:772-778).  For ucm_block_mean it is the
 *               K plane.
 *   repre       one table of block representatives for all layers:
 *               fp32 [n_layers][repre_rows][kv_heads*head_dim]; layer l starts
 *               at repre + l*repre_layer_stride floats.  A request owns the
 *               contiguous rows seg_off[r] .. seg_off[r]+seg_len[r]-1, the
 *               layout of the reference's kpre_caches
 *               (ucm/sparse/gsa/prefetch/prefetch_engine.py:64-77, slots from
 *               ucm/sparse/gsa/gsa.py:188-190).
 */
#ifndef UCM_HIP_H
#define UCM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define UCM_OK 0
#define UCM_EINVAL (-22)
#define UCM_ENOTSUP (-95)
#define UCM_EHIP (-5)
#define UCM_ENOMEM (-12)

#define UCM_DTYPE_F32 0
#define UCM_DTYPE_BF16 1
#define UCM_DTYPE_F16 2

/* ucm_block_mean modes */
#define UCM_MEAN_F32 0       /* fp32 mean kept as is (the C++ KRepreComputer contract) */
#define UCM_MEAN_BF16_ROUND 1 /* mean rounded to bf16 and widened (what the live torch path stores) */
#define UCM_MEAN_BF16_STORE 2 /* the same rounded mean kept as bf16: `repre` is a bf16 table */
#define UCM_MEAN_ABS 4        /* or-ed to one of the above: the mean of the ABSOLUTE values, token order as before
                               (the per-channel |k| statistic KVStar picks its channels by,
                               ucm/sparse/kvstar/multistep.py:284-292, one block at a time) */
#define UCM_MEAN_KEYS_F16 8   /* or-ed to UCM_MEAN_F32 or UCM_MEAN_BF16_ROUND: the key cache is fp16 (a model that runs in
                              * float16), and "rounded" then means rounded to fp16, the cache's own type, and widened.
                              * UCM_MEAN_BF16_STORE is not offered for fp16 caches (UCM_ENOTSUP). */

typedef void* ucm_stream_t; /* hipStream_t */

/* Library version (major*10000 + minor*100 + patch) and the text of the last
 * error raised on the calling thread ("" if none). */
int ucm_version(void);
const char* ucm_last_error(void);

/*
 * Block representatives: mean over the block_size tokens of each listed block,
 * per (kv head, dim), accumulated in fp32 in token order and multiplied by
 * 1/block_size - the arithmetic of KRepreComputer::ComputeKRepreBlock
 * (ucm/sparse/gsa/offload_ops/src/k_repre.cpp:15-35 with VectorMeanImpl,
 * src/vec_product.cpp:39-85), read straight from the paged bf16 key cache the
 * way the live hooks index it (GSA.copy_k, ucm/sparse/gsa/gsa.py:634-654;
 * ReqStatePerLayer.extract_block_repre, ucm/sparse/esa/esa.py:265-266).
 *   k_layers   dev: n_layers pointers to bf16 [num_blocks][block_size][kv_heads][head_dim]
 *              (fp16 with UCM_MEAN_KEYS_F16 or-ed to the mode)
 *   block_ids  dev int32[n]: cache blocks to reduce (same ids in every layer)
 *   slots      dev int32[n]: destination row of each block in `repre`
 *   num_blocks, repre_rows: sizes of a K plane and of one layer's table; an id
 *              or slot outside them is skipped by the kernel, not dereferenced.
 *   repre      dev: fp32 [n_layers][repre_rows][kv_heads*head_dim] for modes
 *              UCM_MEAN_F32 / UCM_MEAN_BF16_ROUND, bf16 of the same shape for
 *              UCM_MEAN_BF16_STORE (the dtype the live path keeps its
 *              representatives in, gsa.py:640-652); repre_layer_stride in
 *              ELEMENTS of that type.
 * Requires kv_heads*head_dim to be a multiple of 8 and 16-byte aligned planes.
 */
int ucm_block_mean(const void* const* k_layers, int n_layers, int num_blocks,
                   const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                   int kv_heads, int head_dim, void* repre, int repre_rows,
                   int64_t repre_layer_stride, int mode, ucm_stream_t stream);

/*
 * Scores of every block of a ragged batch, all layers in one launch:
 *   qbar[h]  = (q[h*g] + q[h*g+1] + ... + q[h*g+g-1]) * (1/g),  g = q_heads/kv_heads
 *   score[b] = sum over kv heads h, in order, of max over r < num_repre of dot(qbar[h], repre[b][h][r])
 * with dot() in the 16-lane FMA + pairwise fold order of the reference's
 * AVX-512 build, so the fp32 results equal TopkBlockSelector::ComputeQHeadMean
 * + ComputeKQDotScores bit for bit
 * (ucm/sparse/gsa/offload_ops/src/select_topk_block.cpp:53-114,
 * src/vec_product.cpp:16-37; the reference configures one representative per
 * head, numKrepre = 1, ucm/sparse/gsa/gsa.py:501).
 *   q          dev: queries, q_dtype fp32, bf16 or fp16, [n_layers][*][q_heads][head_dim];
 *              layer l starts q_layer_stride ELEMENTS after layer l-1; request
 *              r reads row q_rows[r] (q_rows == NULL: row r); with q_rows,
 *              q_layer_stride is also the bound of a layer's rows: a request
 *              whose row lies outside it is skipped, its scores are left as
 *              they were (ucm_hash_encode_queries does the same).  This is the
 *              reference's gsa_q_cache (gsa.py:503-512) when fp32, or the
 *              layer's raw query tensor with q_rows = index of each request's
 *              last token (GSA.copy_q, gsa.py:616-632) in the model dtype.
 *   repre      dev: representative table [n_layers][repre_rows][kv_heads][num_repre][head_dim],
 *              repre_dtype fp32 or bf16 (what ucm_block_mean wrote), layer
 *              stride in ELEMENTS.  A bf16 table is widened exactly, so it
 *              scores like the fp32 table holding the same bf16-rounded means,
 *              at half the bytes streamed.
 *   seg_off, seg_len  dev int32[n_req]: first representative row and number of
 *              blocks of each request; max_seg_len >= every seg_len (host
 *              value, sizes the grid; a longer seg_len is cut there);
 *              total_blocks = sum of seg_len when the host knows it (a tighter
 *              grid), else 0.  These descriptors live in device memory, where
 *              the host cannot check them: a request whose rows do not lie
 *              inside [0, repre_rows) is skipped, its scores left as they were.
 *   scores     dev fp32: score of row x of layer l at scores[l*scores_layer_stride + x];
 *              a layer holds at least repre_rows scores.
 *   scale      every score is multiplied by it on the way out; 1 leaves the bits
 *              above.  1/kv_heads gives the values of the reference's torch
 *              variant, the mean over all q heads of TopkCal.cal_topk
 *              (ucm/sparse/gsa/gsa.py:386-412, to the rounding of its own
 *              summation order; the ranking is the same for any positive scale).
 *   tile_blocks  blocks scored per workgroup; 0 sizes a workgroup's share to 128 KiB
 *              of representatives (a value for benchmarks and tests, not part of
 *              the reference interface).
 * head_dim must be 32, 64, 96, 128, 192 or 256, kv_heads*num_repre one of 1, 2,
 * 4, 8, 16 and kv_heads*num_repre*head_dim at most 2048.
 */
int ucm_score_blocks(const void* q, int q_dtype, int64_t q_layer_stride, const int32_t* q_rows,
                     int q_heads, const void* repre, int repre_dtype, int64_t repre_layer_stride,
                     int64_t repre_rows, int num_repre, const int32_t* seg_off, const int32_t* seg_len,
                     int n_req, int max_seg_len, int64_t total_blocks, int n_layers, int kv_heads,
                     int head_dim, float* scores, int64_t scores_layer_stride, float scale,
                     int tile_blocks, ucm_stream_t stream);

/*
 * Per-request block selection with forced windows, all layers in one launch -
 * TopkBlockSelector::TopKImpl (select_topk_block.cpp:20-51; windows 1 and 2 by
 * default, include/select_topk_block.h:20): if start_w+end_w >= n or k >= n or
 * k == 0 the result is 0..n-1 (n entries); otherwise the first start_w blocks,
 * the k-start_w-end_w best of the rest by score (equal scores: lower index
 * first, as std::stable_sort leaves them) and the last end_w blocks, sorted
 * ascending.  k = topk_len[r] is the total (ucm/sparse/utils.py:30-36).
 *   scores_rows  scores a layer holds: a request whose seg_off .. seg_off+seg_len
 *              does not lie inside [0, scores_rows) selects nothing (count 0)
 *   idx_out    dev int32: entry j of request r in layer l at
 *              idx_out[(l*n_req + r)*out_stride + j]; out_stride must hold
 *              max(k, n) of every request.
 *   count_out  dev int32[n_layers][n_req]: entries written.
 * Optionally (block_tables != NULL) the logical->physical step of
 * GSAPrefetchBase._no_gsa_input_deal
 * (ucm/sparse/gsa/prefetch/prefetch_engine.py:507-553) is fused in:
 *   block_tables  dev int32[n_req][bt_stride]: cache block id of logical block i
 *   phys_out      dev int32, same layout as idx_out: block_tables[r][idx]
 *   seq_lens      dev int32[n_req] (may be NULL): tokens of each request;
 *   sparse_seq_lens dev int32[n_layers][n_req]: count*block_size, minus
 *              block_size - seq_len%block_size when the last block is partial;
 *              seq_len itself when every block was kept (the reference's
 *              non-sparsified branch, prefetch_engine.py:547-553).
 * Up to 4096 blocks per request.
 */
int ucm_topk_windows(const float* scores, int64_t scores_layer_stride, int64_t scores_rows,
                     const int32_t* seg_off, const int32_t* seg_len, const int32_t* topk_len, int n_req,
                     int max_seg_len, int n_layers, int start_w, int end_w, int32_t* idx_out,
                     int out_stride, int32_t* count_out, const int32_t* block_tables, int bt_stride,
                     int32_t* phys_out, const int32_t* seq_lens, int block_size,
                     int32_t* sparse_seq_lens, ucm_stream_t stream);

/*
 * ucm_score_blocks and ucm_topk_windows as ONE launch - what
 * TopkBlockSelector::SelectTopK does per request (select_topk_block.cpp:116-129:
 * group mean, scores, selection) for every request and layer of the call.  A
 * request's scoring workgroups each take a ticket when their scores are visible
 * to the whole device; the one that draws the last ticket runs the request's
 * selection, so no second launch waits for the first to drain.  Scores and
 * selections are bit-identical to the two calls.
 *
 * The arguments travel in a struct so that a caller that issues the call once
 * per layer (the plugin's attention hook) fills it once per step and changes
 * two fields (q, first_layer) per call.  Fields are those of the two entry
 * points above, with these differences:
 *   struct_size  sizeof(ucm_score_select_args_t), checked
 *   q          the queries of layer first_layer (a layer's own query tensor);
 *              every other pointer names layer 0 of its table, and the call
 *              works on layers first_layer .. first_layer+n_layers-1
 *   repre_rows  rows of a layer of `repre` AND scores a layer of `scores` holds
 *   idx_layer_stride, count_layer_stride  elements between two layers of
 *              idx_out / phys_out and of count_out / sparse_seq_lens / tickets;
 *              0 = dense (n_req*out_stride and n_req).  A caller that keeps
 *              persistent [layers][max_requests][...] tables and runs a batch of
 *              fewer requests names the tables' own strides.
 *   total_blocks  as for ucm_score_blocks (0 = unknown)
 *   tickets    dev int32 [layers][n_req] (indexed like count_out): zero before
 *              the first call; every call leaves it zero.  Calls that overlap
 *              in time (different streams) need arrays of their own.
 * Up to 1024 blocks per request (UCM_ENOTSUP beyond: use the two calls).
 */
typedef struct ucm_score_select_args {
    size_t struct_size;
    const void* q;
    int q_dtype;
    int q_heads;
    int64_t q_layer_stride;
    const int32_t* q_rows;
    const void* repre;
    int repre_dtype;
    int num_repre;
    int64_t repre_layer_stride;
    int64_t repre_rows;
    const int32_t* seg_off;
    const int32_t* seg_len;
    const int32_t* topk_len;
    int n_req;
    int max_seg_len;
    int first_layer;
    int n_layers;
    int kv_heads;
    int head_dim;
    float* scores;
    int64_t scores_layer_stride;
    float scale;
    int tile_blocks;
    int start_w;
    int end_w;
    int32_t* idx_out;
    int32_t* count_out;
    int out_stride;
    int bt_stride;
    const int32_t* block_tables;
    int32_t* phys_out;
    const int32_t* seq_lens;
    int32_t* sparse_seq_lens;
    int block_size;
    int reserved;
    int32_t* tickets;
    int64_t idx_layer_stride;
    int64_t count_layer_stride;
    int64_t total_blocks;
} ucm_score_select_args_t;
int ucm_score_select(const ucm_score_select_args_t* args, ucm_stream_t stream);

/*
 * The ESA retrieval backend's computation for a batch of requests -
 * RetrievalWorkerBackend::worker_loop
 * (ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp:135-203): for request b,
 * every entry of indexes[b][0..m) that is not -1 names a row of `data`
 * (fp32 [n_items][dim], the table the backend is constructed over, :19-26); its
 * score is the strictly sequential sum over d of q[b][d]*data[row][d] with
 * separately rounded multiply and add (:175-181); the min(valid entries, topk)
 * best are returned in descending score order with their scores (:182-189).
 * Equal scores come out in index-row order (the reference's std::partial_sort
 * leaves that order unspecified).  Entries that are -1 or outside
 * [0, n_items) are skipped.
 *   q          dev fp32 [batch][dim]
 *   indexes    dev int32 [batch][m], padded with -1 (submit(), :43-74)
 *   scores_ws  dev fp32 [batch][m]: workspace for all candidate scores
 *   out_idx / out_scores  dev [batch][out_stride]; out_count dev int32[batch]
 * dim must be a multiple of 4, m at most 8192.
 */
int ucm_esa_retrieve(const float* data, int n_items, int dim, const float* q,
                     const int32_t* indexes, int batch, int m, int topk, float* scores_ws,
                     int32_t* out_idx, float* out_scores, int32_t* out_count, int out_stride,
                     ucm_stream_t stream);

/*
 * ucm_esa_retrieve over a persistent table of requests: the plugin keeps one
 * row per live request (its slot list, ReqStatePerLayer.slots,
 * ucm/sparse/esa/esa.py:170-175,358-362) in device memory and each call
 * covers the requests that retrieve in this step
 * (ReqStatePerLayer.start_retrieval, esa.py:286-301, for all of a layer's
 * requests at once instead of one submit per request).
 *   slot_table  dev int32 [table_rows][table_stride], -1 padded: row i = slot
 *               list of the request that owns row i; only its first m entries
 *               are looked at (m = the longest list among this call's
 *               requests, so short batches do not pay for the table's width)
 *   rows        dev int32 [batch]: table row of request b of this call (q is
 *               [batch][dim], scores_ws [batch][m]); a row outside the table
 *               makes that request a no-op
 *   topk_rows   dev int32 [table_rows]: each request's own k (at most max_topk)
 *   out_idx / out_pos / out_scores  dev [table_rows][out_stride], out_count dev
 *               int32 [table_rows]: results of request b go to row rows[b], so
 *               they stay with the request until a later step consumes them.
 *               out_pos (may be NULL) is the winner's position in its slot
 *               list, i.e. the block's index relative to the request
 *               (slots_to_relative_indexes, esa.py:358-361) - what
 *               ucm_delta_plan_rows takes as `sel`.
 */
int ucm_esa_retrieve_rows(const float* data, int n_items, int dim, const float* q,
                          const int32_t* slot_table, int table_rows, int table_stride, int m,
                          const int32_t* rows, int batch, const int32_t* topk_rows, int max_topk,
                          float* scores_ws, int32_t* out_idx, int32_t* out_pos, float* out_scores,
                          int32_t* out_count, int out_stride, ucm_stream_t stream);

/*
 * ucm_esa_retrieve for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): it has no
 * counterpart in the reference.  Same arguments and results as
 * ucm_esa_retrieve, minus scores_ws: the candidate scores go to a scratch
 * array that is part of the library image (2 MiB per GPU, held until the
 * process ends), so the call allocates nothing.  batch*m may be at most
 * 524288 (2^19) candidate scores; a larger call fails with UCM_ENOTSUP.
 * The first call on a GPU looks the array's device address up (no allocation).
 * All calls on one GPU share the array: two of them that overlap in time (on
 * different streams or from different threads) race; calls that follow one
 * another on a stream do not.  Nothing in the array has to be cleared
 * between calls (every score a call reads it has written itself).
 */
int ucm_esa_retrieve_static(const float* data, int n_items, int dim, const float* q,
                            const int32_t* indexes, int batch, int m, int topk, int32_t* out_idx,
                            float* out_scores, int32_t* out_count, int out_stride,
                            ucm_stream_t stream);

/*
 * Delta loads: decides, per (layer, request), which staging slots keep their
 * block and which missing block of the new selection goes where - the
 * "load delta" of ReqStatePerLayer.wait_retrieval_and_start_load
 * (ucm/sparse/esa/esa.py:312-338; the hit / miss / evict sets of
 * GSAPrefetchEngineC::GetHitAndMissBlock, ucm/sparse/gsa/prefetch/src/kvcache_pre.cpp:206-238)
 * computed on the device from ucm_topk_windows' output.  A block is identified
 * by its logical index within the request.
 *   sel, sel_phys  dev int32 [n_layers][n_req][sel_stride]: selected logical
 *                  blocks and their cache block ids (idx_out / phys_out)
 *   count          dev int32 [n_layers][n_req]: entries of sel that are valid
 *   resident       dev int32 [n_layers][n_req][n_slots], in/out: logical block
 *                  held by each staging slot, -1 = empty
 *   load_phys      dev int32 [n_layers][n_req][n_slots], out: cache block id to
 *                  copy into the slot, -1 = slot untouched.  It is exactly the
 *                  `phys` argument of ucm_kv_gather_selected (count = n_slots),
 *                  which skips the -1 entries.
 *   slot_of_sel    dev int32, layout of sel, out: staging slot that holds each
 *                  selected block after the load (the sparse block table)
 *   miss_count     dev int32 [n_layers][n_req], out: blocks to load
 * The i-th missing block (ascending) goes to the i-th freed slot (ascending);
 * the reference pairs them in set order, which is unspecified.  At most 1024
 * slots per request and layer (one wave up to 64 slots, a 256-thread workgroup
 * beyond); selections longer than n_slots are cut there.
 */
int ucm_delta_plan(const int32_t* sel, const int32_t* sel_phys, const int32_t* count, int n_req,
                   int n_layers, int sel_stride, int32_t* resident, int n_slots, int32_t* load_phys,
                   int32_t* slot_of_sel, int32_t* miss_count, ucm_stream_t stream);

/*
 * ucm_delta_plan over a persistent table of requests: every array is laid out
 * [n_layers][table_rows][...] and request b of the call uses row rows[b] (dev
 * int32 [batch]); rows outside the table are skipped.  With sel_phys == sel
 * the plan's load_phys holds the logical block each slot is to receive, which
 * is what ucm_kv_load_planned reads.
 */
int ucm_delta_plan_rows(const int32_t* sel, const int32_t* sel_phys, const int32_t* count,
                        const int32_t* rows, int batch, int table_rows, int n_layers, int sel_stride,
                        int32_t* resident, int n_slots, int32_t* load_phys, int32_t* slot_of_sel,
                        int32_t* miss_count, ucm_stream_t stream);

/*
 * The bookkeeping of the GSA prefetch engine for a batch of requests, all
 * layers in one launch - GSAPrefetchEngineC::RunOneBsPrefetch with
 * GetHitAndMissBlock, RunPrefetchH2D and LoadKVToHBM
 * (ucm/sparse/gsa/prefetch/src/kvcache_pre.cpp:206-322).  Per (request, layer):
 * selected logical blocks that a resident cache block holds are hits, the
 * others misses (in selection order); the free list is walked in order, entries
 * whose block became a hit are passed over, every other takes the next miss and
 * from then on holds that logical block; the success table lists the cache
 * blocks of hits and served misses by logical index ascending (the row is
 * zeroed first); the free list is rebuilt from the resident blocks outside the
 * hit set by block id ascending.
 *   map_block  dev int32 [table_rows][cap]: cache block of each resident slot of
 *              a request (mBlocksMap's keys; the same in every layer), map_len
 *              dev int32 [table_rows] slots in use
 *   map_idx    dev int32 [n_layers][table_rows][cap], in/out: logical block each
 *              slot holds (mBlocksMap's values; mDocsTables is the inverse)
 *   topk_idx   dev int32 [n_layers][batch][topk_stride], topk_len dev int32
 *              [batch]: the selections (mUseTopkIdxs, topkLensInput)
 *   rows, bs_index  dev int32 [batch]: table row and batch slot of request i; a
 *              request with topk_len <= 0 or a row outside the table is skipped
 *              (CallPrefetchProcessFun, :376-381)
 *   free_block / free_len      dev int32 [n_layers][max_bs][row_len] / [n_layers][max_bs], in/out (mFreeBlock)
 *   success_blocks / success_len  the same shapes, out (mLoadSuccessBlocks, mSuccessTableLen)
 *   load_blocks  dev int32 [n_layers][table_rows][cap], load_count dev int32
 *              [n_layers][table_rows]: cache blocks that receive a load, in order
 *              (allNeedLoadBlock, kept with the request's row);
 *              miss_idxs dev int32 [n_layers][table_rows][topk_stride], miss_count:
 *              ALL misses in selection order (allMissIdxs); load_blocks[j]
 *              receives logical block miss_idxs[j].  With load_sel = miss_idxs,
 *              dst_table = load_blocks and load_count they are the arguments of
 *              ucm_kv_load_planned.
 * A selection names a logical block once and the free list a block once, both
 * blocks of the map (what the reference's Python side guarantees).  At most 256
 * resident blocks, selected blocks and free-list entries per request.
 */
int ucm_prefetch_plan(const int32_t* map_block, const int32_t* map_len, int32_t* map_idx, int table_rows,
                      int cap, const int32_t* topk_idx, int topk_stride, const int32_t* topk_len,
                      const int32_t* rows, const int32_t* bs_index, int batch, int n_layers, int max_bs,
                      int row_len, int32_t* free_block, int32_t* free_len, int32_t* success_blocks,
                      int32_t* success_len, int32_t* load_blocks, int32_t* load_count, int32_t* miss_idxs,
                      int32_t* miss_count, ucm_stream_t stream);

/*
 * Hash-code retrieval (KvComp).  A vector's code has bit c = (x . W[:, c] > 0),
 * packed LSB first (bit j of byte b is column 8b+j) - HashEncoder.compute_hash
 * (ucm/sparse/kvcomp/hash_encoder.py:99-157, bit order :92-97,139-149; W is
 * [head_dim][bits] in the model dtype, :65-71).  The sign is that of the exactly
 * accumulated product (matrix cores, with an fp64 redo of every result inside
 * the fp32 error bound).  head_dim = bits = 128.
 *
 * ucm_hash_encode_blocks: codes of the keys of the listed cache blocks
 * (ReqStatePerLayer.extract_block_repre, ucm/sparse/kvcomp/kvcomp.py:314-347),
 * read from the paged bf16 key cache like ucm_block_mean reads it.  Per block:
 *   token_codes  dev u8 [n_layers][rows][block_size][kv_heads][16] (cache order;
 *                may be NULL), layer stride in BYTES
 *   colsum       dev int16 [n_layers][rows][kv_heads][128]: #ones - #zeros of
 *                each bit over the block's tokens, layer stride in ELEMENTS
 *   block_codes  dev u8 [n_layers][rows][kv_heads][16]: majority vote of each bit
 *                (colsum > 0; an exact tie gives 0), layer stride in BYTES
 *   workgroups   persistent workgroups launched over all layers, each of whose
 *                waves steps through the list of blocks; 0 = the default (4096)
 * A block is encoded in tiles of 32 key vectors: block_size * kv_heads must be
 * a multiple of 32 (UCM_ENOTSUP otherwise; 16-token blocks need two kv heads
 * or more), kv_heads one of 1, 2, 4, 8 and block_size at most 16383.
 * ucm_hash_encode_queries: per (layer, request) the codes of all query heads
 * (q_codes u8 [L][n_req][q_heads][16]), their +-1 sum over heads (q_sum int16
 * [L][n_req][128]) and the code of every kv head's group-mean query
 * (qbar_codes u8 [L][n_req][kv_heads][16]); q is bf16 laid out as for
 * ucm_score_blocks.
 * ucm_hash_score_blocks: fp32 scores of all blocks of a ragged batch, written
 * where ucm_topk_windows reads them.
 *   mode 0  the reference's score (kvcomp.py:237-247): the sum over query heads,
 *           kv heads and the block's tokens of the +-1 inner products, computed
 *           as <q_sum, sum_h colsum[h]> (the same integer); round_fp16 != 0
 *           rounds it to fp16 as the reference's fp16 sum does.
 *   mode 1  sum over kv heads of (128 - hamming(qbar code, majority block code)),
 *           the benchmark's block-code variant (not present in the reference);
 *           qbar_codes, block_codes and block_codes_layer_stride must be
 *           multiples of 16 bytes (UCM_EINVAL otherwise): a kv head's code is
 *           read as one 16-byte load.
 *   rows    rows of a layer of the summary tables (colsum / block_codes) and of
 *           `scores`: a request whose seg_off .. seg_off+seg_len does not lie inside
 *           [0, rows) is not scored (its descriptors live in device memory).
 * The reference keeps init 1 / local 2 blocks out of the candidates and
 * index-sorts its picks (kvcomp.py:219-221,249-254): ucm_topk_windows with the
 * matching windows gives the same set.
 */
int ucm_hash_encode_blocks(const void* const* k_layers, int n_layers, int num_blocks,
                           const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                           int kv_heads, int head_dim, const void* w_bf16, int bits, int rows,
                           uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                           int64_t colsum_layer_stride, uint8_t* block_codes,
                           int64_t block_codes_layer_stride, int workgroups, ucm_stream_t stream);
int ucm_hash_encode_queries(const void* q_bf16, int64_t q_layer_stride, const int32_t* q_rows,
                            int n_req, int n_layers, int q_heads, int kv_heads, int head_dim,
                            const void* w_bf16, int bits, uint8_t* q_codes, int16_t* q_sum,
                            uint8_t* qbar_codes, ucm_stream_t stream);
/*
 * The same two calls for a float16 model: keys (or queries) and weights are float16 - HashEncoder draws its weights
 * in the model's type (ucm/sparse/kvcomp/hash_encoder.py:65-71) - and the codes are the signs of the exactly
 * accumulated float16 products.  With several query heads per kv head the group means are fp32 numbers, as in the
 * bf16 call, and the mean codes are the signs of their exactly accumulated products with the float16 weights.
 */
int ucm_hash_encode_blocks_f16(const void* const* k_layers, int n_layers, int num_blocks,
                               const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                               int kv_heads, int head_dim, const void* w_f16, int bits, int rows,
                               uint8_t* token_codes, int64_t token_codes_layer_stride, int16_t* colsum,
                               int64_t colsum_layer_stride, uint8_t* block_codes,
                               int64_t block_codes_layer_stride, int workgroups, ucm_stream_t stream);
int ucm_hash_encode_queries_f16(const void* q_f16, int64_t q_layer_stride, const int32_t* q_rows,
                                int n_req, int n_layers, int q_heads, int kv_heads, int head_dim,
                                const void* w_f16, int bits, uint8_t* q_codes, int16_t* q_sum,
                                uint8_t* qbar_codes, ucm_stream_t stream);
int ucm_hash_score_blocks(int mode, const int16_t* q_sum, const uint8_t* qbar_codes,
                          const int16_t* colsum, int64_t colsum_layer_stride,
                          const uint8_t* block_codes, int64_t block_codes_layer_stride, int64_t rows,
                          const int32_t* seg_off, const int32_t* seg_len, int n_req,
                          int64_t total_blocks, int n_layers, int kv_heads, int bits, float* scores,
                          int64_t scores_layer_stride, int round_fp16, ucm_stream_t stream);

/*
 * KVStar multi-query softmax-vote retrieval.
 *
 * ucm_kvstar_block_repre: the sub-block representatives of
 * ReqPerLayerState.extract_block_repre (ucm/sparse/kvstar/multistep.py:279-316)
 * read straight from the paged bf16 key cache: each listed block is cut into
 * M = block_size/merge sub-blocks, the `merge` tokens of a sub-block are
 * averaged per (kv head, kept channel) - fp32 sum in token order, *(1/merge),
 * rounded to bf16 (the model dtype the reference's mean() returns) and stored
 * as fp16 (its .to(torch.float16), :495-497).
 *   pruned   dev int32[kv_heads][d_pruned]: channel of every kept dim (the
 *            reference's d_pruned_index, :288-304), or NULL when d_pruned ==
 *            head_dim; layer l reads the lists pruned_layer_stride elements
 *            after layer l-1's (the reference picks the channels per layer
 *            state; 0 = one set of lists for every layer), so one launch
 *            covers all layers
 *   pruned_sel  dev int32[n] or NULL: with it a layer has n_pruned_lists
 *            lists ([n_pruned_lists][kv_heads][d_pruned]) and listed block i is
 *            pruned by list pruned_sel[i] - the blocks of several requests,
 *            each with channels of its own, in one launch (a block that names
 *            a list outside [0, n_pruned_lists) is skipped); NULL: list 0
 *   repre    dev fp16 cells of [d_pad/8][M][8] - the 16-byte pieces (8
 *            channels) of a block's M sub-blocks side by side - one per
 *            (layer, kv head, row): cell (l, h, r) starts l*repre_layer_stride
 *            + h*repre_head_stride + r*repre_row_stride elements in.  Cells
 *            must not overlap: either head planes ([kv_heads][repre_rows]
 *            [cell], head stride >= repre_rows * row stride) or the heads of
 *            a row next to each other ([repre_rows][kv_heads][cell], row
 *            stride >= kv_heads * head stride); the two measure the same,
 *            building and reading.  d_pad >=
 *            d_pruned, a multiple of 8 (16 for ucm_kvstar_votes), columns
 *            past d_pruned are written as zero; all strides are multiples of
 *            8.  (The reference keeps [row][M][kv head][d]; inside a cell
 *            every load instruction of the score kernel is a run of whole
 *            cache lines.)
 *
 * ucm_kvstar_votes: the arithmetic of KVStar::Execute
 * (ucm/sparse/kvstar/retrieve/core/domain/retrieve_task/simd_compute_kernel.cpp:817-990)
 * for n_tasks (request, layer) tasks in one go: scores of n_tokens x q_heads
 * query rows against all sub-block representatives of the task, softmax of
 * every row over the task's sub-blocks, votes[block] = sum over rows and over
 * the block's sub-blocks of the probabilities.  The top-k of the votes is
 * taken by ucm_kvstar_topk.  fp32 on the matrix cores;
 * agrees with the reference's scalar loop to rounding, not bit for bit.
 *   q_f16    dev fp16 buffer of q_elems elements; task t's
 *            [n_tokens][q_heads][d_orig] block starts q_off[t] elements in
 *            (dev int64[n_tasks])
 *   pruned   dev int32[n_pruned_lists][kv_heads][d_pruned] channel lists,
 *            pruned_sel dev int32[n_tasks] picks one per task (-1: none); both
 *            NULL when d_pruned == d_orig
 *   repre_f16  dev fp16, one layer of the table above: cell (h, r) starts
 *            h*repre_head_stride + r*repre_row_stride elements in, r < repre_rows;
 *            task t owns rows seg_off[t] .. seg_off[t]+seg_len[t]-1; max_blocks >=
 *            every seg_len (a longer one is cut there)
 *   ws_max, ws_part  dev fp32 scratch of the sizes ucm_kvstar_workspace_floats
 *            returns (rows_per_head = n_tokens * q_heads/kv_heads); votes dev
 *            fp32 [>= repre_rows], task t's votes at votes[seg_off[t] + b].
 * q_off, pruned_sel, seg_off and seg_len live in device memory, where the host
 * cannot check them: a task whose query block does not lie inside the buffer,
 * whose rows do not lie inside [0, repre_rows) or whose list index is not below
 * n_pruned_lists is skipped by every kernel of the call (its votes stay as
 * they were).
 * n_tokens * (q_heads/kv_heads) <= 64, kv_heads <= 8, d_pad a multiple of 16
 * and <= 128, sub_blocks a power of two up to 128.
 */
int ucm_kvstar_block_repre(const void* const* k_layers, int n_layers, int num_blocks,
                           const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                           int kv_heads, int head_dim, int merge, const int32_t* pruned,
                           int64_t pruned_layer_stride, const int32_t* pruned_sel, int n_pruned_lists,
                           int d_pruned, int d_pad, void* repre_f16, int repre_rows,
                           int64_t repre_layer_stride, int64_t repre_head_stride, int64_t repre_row_stride,
                           ucm_stream_t stream);
/* The same for a cache of key_dtype UCM_DTYPE_BF16 (what ucm_kvstar_block_repre takes) or UCM_DTYPE_F16: a float16
 * model's means are rounded once, to float16 (the .mean(dim=2) in the model's type, ucm/sparse/kvstar/multistep.py:310-314;
 * the .to(torch.float16) that follows, :494-499, then changes nothing). */
int ucm_kvstar_block_repre_keys(const void* const* k_layers, int key_dtype, int n_layers, int num_blocks,
                                const int32_t* block_ids, const int32_t* slots, int n, int block_size,
                                int kv_heads, int head_dim, int merge, const int32_t* pruned,
                                int64_t pruned_layer_stride, const int32_t* pruned_sel, int n_pruned_lists,
                                int d_pruned, int d_pad, void* repre_f16, int repre_rows,
                                int64_t repre_layer_stride, int64_t repre_head_stride, int64_t repre_row_stride,
                                ucm_stream_t stream);
/*
 * The query tokens a step contributes to its requests' retrieval groups, copied aside as fp16 - save_to_standby
 * (ucm/sparse/kvstar/multistep.py:318-324, one clone per request and layer) together with the .to(float16) of
 * retrieval_async (:252-254), for all requests of a layer in one launch:
 *   ring_f16[dst_off[i] .. dst_off[i]+row_elems) = fp16(q[src_rows[i]][0 .. row_elems))
 *   q          dev: [q_rows][row_elems] fp32, bf16 or fp16 (a layer's query tensor, row_elems = q_heads*head_dim)
 *   src_rows   dev int32[n], dst_off dev int64[n] (elements into the ring, multiples of 8)
 * A row outside [0, q_rows) or a place outside [0, ring_elems) is skipped.  The groups then are the `q_f16`
 * of ucm_kvstar_votes with q_off pointing into the ring.
 */
int ucm_kvstar_park_queries(const void* q, int q_dtype, int64_t q_rows, int row_elems, const int32_t* src_rows,
                            const int64_t* dst_off, int n, void* ring_f16, int64_t ring_elems, ucm_stream_t stream);

/* ucm_kvstar_votes has two paths: one workgroup per (task, kv head) that keeps
 * the task's per-(block, query row) sums in LDS and stores only the head's
 * share of the votes (taken when there are at least 128 such pairs and the
 * plane fits 159 KiB), and a workspace path that may cut a task into chunks.
 * tiles_per_wave > 0: the workspace path with that many 32-sub-block tiles per
 * wave (four waves per workgroup); -1: the in-LDS path whenever the plane
 * fits; 0: automatic (what callers other than benchmarks and tests pass).
 *
 * ucm_kvstar_workspace_floats: floats of scratch ucm_kvstar_votes[_tables]
 * needs for a call of this shape and tiles_per_wave (rows_per_head = n_tokens *
 * q_heads/kv_heads); the in-LDS path only needs room for the kv heads' vote
 * shares.  The votes calls take the sizes of the two areas (ws_max_floats,
 * ws_part_floats) and fail with UCM_EINVAL when the path they would take needs
 * more. */
int ucm_kvstar_workspace_floats(int n_tasks, int kv_heads, int rows_per_head, int max_blocks,
                                int sub_blocks, int d_pad, int tiles_per_wave, int64_t* max_floats,
                                int64_t* part_floats);
int ucm_kvstar_votes(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads,
                     int d_orig, const int32_t* pruned, int n_pruned_lists, const int32_t* pruned_sel,
                     const void* repre_f16, int64_t repre_rows, int64_t repre_head_stride,
                     int64_t repre_row_stride, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                     int max_blocks, int sub_blocks, int kv_heads, int d_pruned, int d_pad, float* ws_max,
                     int64_t ws_max_floats, float* ws_part, int64_t ws_part_floats, float* votes,
                     int tiles_per_wave, ucm_stream_t stream);
/* The same for tasks whose representatives do not share one table (the
 * reference keeps one blk_repre tensor per request and layer,
 * ucm/sparse/kvstar/multistep.py:191,483-501): task t's table starts at
 * task_tables[t] (dev array of n_tasks dev pointers, 16-byte aligned; cell
 * (h, r) of task t's table starts h*task_head_strides[t] + r*task_row_stride
 * elements in, multiples of 8) and its block 0 is the table's row 0; seg_off
 * only places the task's votes, inside votes[0 .. votes_rows) (a task whose
 * votes would fall outside is skipped; the table pointers themselves are
 * addresses the caller vouches for). */
int ucm_kvstar_votes_tables(const void* q_f16, int64_t q_elems, const int64_t* q_off, int n_tokens, int q_heads,
                            int d_orig, const int32_t* pruned, int n_pruned_lists, const int32_t* pruned_sel,
                            const void* const* task_tables, const int64_t* task_head_strides,
                            int64_t task_row_stride, const int32_t* seg_off, const int32_t* seg_len, int n_tasks,
                            int max_blocks, int sub_blocks, int kv_heads, int d_pruned, int d_pad, float* ws_max,
                            int64_t ws_max_floats, float* ws_part, int64_t ws_part_floats, float* votes,
                            int64_t votes_rows, int tiles_per_wave, ucm_stream_t stream);

/*
 * The selection step of KVStar::Execute on the votes of n_tasks tasks
 * (simd_compute_kernel.cpp:955-977): a min-heap of (score, block) pairs that
 * blocks enter in index order and that, once it holds topk pairs, replaces its
 * smallest pair only for a strictly greater score.  Which of several blocks
 * tied at the k-th score survive follows that process exactly (not the
 * lowest-index rule of ucm_topk_windows).  idx_out[t*out_stride + j] holds the
 * chosen blocks of task t in ASCENDING index order, count_out[t] =
 * min(topk_len[t], seg_len[t]) of them; the reference returns them descending
 * by (score, index), an order the caller restores by sorting these few
 * entries.  votes as written by ucm_kvstar_votes (task t's at
 * votes[seg_off[t] + b], inside votes[0 .. votes_rows): a task outside selects
 * nothing); topk_len[t] >= 1; at most 4096 blocks per task.
 */
int ucm_kvstar_topk(const float* votes, int64_t votes_rows, const int32_t* seg_off, const int32_t* seg_len,
                    const int32_t* topk_len, int n_tasks, int max_seg_len, int32_t* idx_out,
                    int out_stride, int32_t* count_out, ucm_stream_t stream);

/*
 * The order in which KVStar::Execute hands the chosen blocks back
 * (simd_compute_kernel.cpp:969-977: the heap is emptied smallest pair first
 * and the list reversed, so blocks come out descending by (score, index)),
 * restored in place on ucm_kvstar_topk's output: afterwards
 * idx_io[t*out_stride + j], j < count[t], is the j-th block the reference
 * returns for task t.  The reference's caller loads the j-th block into the
 * request's j-th candidate cache block (ucm/sparse/kvstar/multistep.py:410-450),
 * so with this order ucm_kv_load_planned can follow the list without a host
 * round trip.  votes, seg_off, seg_len as for ucm_kvstar_topk; count dev
 * int32[n_tasks] (its count_out); max_count >= every count, at most 4096.
 */
int ucm_kvstar_order(const float* votes, int64_t votes_rows, const int32_t* seg_off, const int32_t* seg_len,
                     int n_tasks, int max_count, int32_t* idx_io, int out_stride, const int32_t* count,
                     ucm_stream_t stream);

/*
 * `num` independent copies of `size` bytes, dst[i] <- src[i]: the batched
 * pointer-array copy of the reference's device layer (H2DKernel / D2HKernel,
 * ucm/store/device/cuda/cuda_device.cu:47-81, reached through
 * H2DBatchSync / D2HBatchSync :180-211).  dst/src are dev arrays of `num`
 * pointers; size and every pointer must be multiples of 16.
 */
int ucm_copy_batch(void* const* dst, const void* const* src, size_t num, size_t size,
                   ucm_stream_t stream);

/*
 * Rows of one array copied into rows of another: dst[dst_idx[i]] <- src[src_idx[i]],
 * i < n, `row_bytes` each.  This is copy_q of the reference's GSA
 * (ucm/sparse/gsa/gsa.py:616-632, `gsa_q_cache[layer][:len(ids)].copy_(query[ids])`):
 * the last query token of every request of a layer kept for the selection that
 * the next step applies.  src is [src_rows][row_bytes], dst [dst_rows][row_bytes],
 * both dev and 16-byte aligned, row_bytes a multiple of 16; src_idx dev int32[n];
 * dst_idx dev int32[n] or NULL (row i).  A pair with either index outside its
 * array is skipped.  Destination rows named twice get one of the sources.
 */
int ucm_park_rows(const void* src, int64_t src_rows, const int32_t* src_idx, void* dst, int64_t dst_rows,
                  const int32_t* dst_idx, int n, size_t row_bytes, ucm_stream_t stream);

/*
 * Transfer device of the store layer: the HIP counterpart of the reference's
 * IDevice (ucm/store/device/idevice.h:33-58) as implemented by CudaDevice on
 * the buffered base (ucm/store/device/cuda/cuda_device.cu:107-227,
 * ucm/store/device/ibuffered_device.h:32-66).  One object per GPU and user:
 * it owns a stream of default priority, `buffer_number` pinned host buffers of
 * `buffer_size` bytes each and the device scratch of the batched copies.
 *
 * ucm_device_create             Setup(): selects the device, allocates the pool
 *                               and the stream (cuda_device.cu:113-125).
 * ucm_device_get_buffer         GetBuffer(size): a free pool slot if size fits
 *                               one and one is free, else a pinned buffer of its
 *                               own (ibuffered_device.h:48-62); NULL on failure.
 * ucm_device_release_buffer     what dropping the reference's shared_ptr does:
 *                               the slot goes back to the pool, a buffer of its
 *                               own is freed.
 * ucm_device_h2d_sync/d2h_sync  H2DSync / D2HSync (cuda_device.cu:126-133).
 * ucm_device_h2d_async/d2h_async  H2DAsync / D2HAsync on the object's stream
 *                               (:134-141).
 * ucm_device_append_callback    AppendCallback (:142-156): cb(ok, user) runs on
 *                               a runtime thread once everything queued before it
 *                               on the stream has finished; ok is 1 on success.
 *                               The callback must not call this library.
 * ucm_device_synchronized       Synchronized (:157-160): waits for the stream.
 * ucm_device_h2d_batch_sync     H2DBatchSync (:180-195): `number` copies of
 *                               `count` bytes, device dArr[i] <- host hArr[i].
 * ucm_device_d2h_batch_sync     D2HBatchSync (:196-211): host hArr[i] <- device
 *                               dArr[i].  Both arrays are HOST arrays of
 *                               addresses (as in the reference).  One launch of
 *                               the ucm_copy_batch kernel on the object's
 *                               stream, then a wait, when every address is
 *                               memory a kernel can touch (device memory,
 *                               pinned host memory such as this object's
 *                               buffers) and `count` and the addresses are
 *                               multiples of 16; otherwise (pageable host
 *                               memory included) one runtime copy per pair.
 * ucm_device_stream             the object's stream, for callers that order
 *                               their own kernels against the copies.
 *
 * Calls on one object may come from several threads; batched copies on one
 * object run one at a time.
 */
/* 1 if a kernel of this library may dereference [address, address + count):
 * device memory, pinned or registered host memory, managed memory; 0 for
 * pageable host memory, unknown addresses and NULL.  Callers that pass raw
 * addresses to ucm_copy_batch (as the store's fetch_data / dump_data do,
 * ucm/store/ucmstore.py:127-167) check them with it: a kernel that touches
 * pageable memory faults. */
int ucm_kernel_can_access(const void* address, size_t count);

typedef struct ucm_device ucm_device_t;
typedef void (*ucm_device_callback_t)(int ok, void* user);
int ucm_device_create(int device_id, size_t buffer_size, size_t buffer_number, ucm_device_t** out);
void ucm_device_destroy(ucm_device_t* dev);
void* ucm_device_get_buffer(ucm_device_t* dev, size_t size);
void ucm_device_release_buffer(ucm_device_t* dev, void* buffer);
int ucm_device_h2d_sync(ucm_device_t* dev, void* dst, const void* src, size_t count);
int ucm_device_d2h_sync(ucm_device_t* dev, void* dst, const void* src, size_t count);
int ucm_device_h2d_async(ucm_device_t* dev, void* dst, const void* src, size_t count);
int ucm_device_d2h_async(ucm_device_t* dev, void* dst, const void* src, size_t count);
int ucm_device_append_callback(ucm_device_t* dev, ucm_device_callback_t cb, void* user);
int ucm_device_synchronized(ucm_device_t* dev);
int ucm_device_h2d_batch_sync(ucm_device_t* dev, void* const* d_arr, const void* const* h_arr,
                              size_t number, size_t count);
int ucm_device_d2h_batch_sync(ucm_device_t* dev, void* const* h_arr, const void* const* d_arr,
                              size_t number, size_t count);
ucm_stream_t ucm_device_stream(ucm_device_t* dev);

/*
 * Whole-block dump (cache -> staging) and load (staging -> cache) driven by a
 * list of cache block ids - launch_transfer_task's "dump"/"load"
 * (ucm/sparse/esa/esa.py:222-263, ucm/sparse/gsa/gsa.py:518-560) without one
 * tensor view and one memcpy per block.  Staging block i is in the stored-block
 * format of get_offset (esa.py:124-135, tp_size 1): [layer][K|V] slices of
 * block_bytes each, i.e. slice (i, l, kv) at ((i*n_layers + l)*2 + kv)*block_bytes.
 * block_bytes, kv_stride and all base pointers must be multiples of 16.
 * num_blocks is the number of blocks of one K (or V) plane; an id outside
 * [0, num_blocks) is skipped by the kernel instead of being dereferenced.
 */
int ucm_kv_gather_blocks(const void* const* layers, int n_layers, size_t kv_stride,
                         size_t block_bytes, int num_blocks, const int32_t* block_ids, int n,
                         void* staging, ucm_stream_t stream);
int ucm_kv_scatter_blocks(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                          int num_blocks, const int32_t* block_ids, int n, const void* staging,
                          ucm_stream_t stream);

/*
 * The same moves, and ucm_kv_load_planned below, for one rank of a
 * tensor-parallel group whose ranks share the stored block: get_offset
 * (ucm/sparse/esa/esa.py:124-135) puts rank r's K slice of layer l at
 * 2*block_bytes*tp_size*l + 2*block_bytes*r and its V slice block_bytes later
 * (block_bytes = the rank's own slice: block_size x its kv heads x head_dim),
 * so a stored (or staging) block is n_layers*2*block_bytes*tp_size bytes and a
 * rank touches only its own slices.  0 <= rank < tp_size; (0, 1) is the plain
 * entry point.
 */
int ucm_kv_gather_blocks_tp(const void* const* layers, int n_layers, size_t kv_stride,
                            size_t block_bytes, int num_blocks, const int32_t* block_ids, int n,
                            void* staging, int rank, int tp_size, ucm_stream_t stream);
int ucm_kv_scatter_blocks_tp(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                             int num_blocks, const int32_t* block_ids, int n, const void* staging,
                             int rank, int tp_size, ucm_stream_t stream);

/*
 * Gather of the blocks chosen by ucm_topk_windows, straight from its device
 * output (no host round trip): request r's region of `staging` starts at
 * dst_off[r] blocks and holds [layer][K|V][region_k[r]] blocks, of which the
 * first count[l][r] are written.  The reference moves the same blocks one
 * tensor view at a time (esa.py:254-258).
 *   phys   dev int32[n_layers][n_req][phys_stride], count dev int32[n_layers][n_req]
 *   dst_off dev int64[n_req], region_k dev int32[n_req]; max_count >= every count.
 *   staging_blocks  blocks the staging buffer holds: dst_off and region_k live
 *                   in device memory, where the host cannot check them, so a
 *                   destination at or past this bound is skipped, never written.
 */
int ucm_kv_gather_selected(const void* const* layers, int n_layers, size_t kv_stride,
                           size_t block_bytes, int num_blocks, const int32_t* phys,
                           const int32_t* count, int n_req, int phys_stride, const int64_t* dst_off,
                           const int32_t* region_k, int max_count, void* staging,
                           int64_t staging_blocks, ucm_stream_t stream);

/*
 * The "load" of ReqStatePerLayer.wait_retrieval_and_start_load
 * (ucm/sparse/esa/esa.py:312-339 -> launch_transfer_task :222-263 ->
 * store.load(block_hashes, offsets, [k_cache[id] ...])) when the store's blocks
 * are device-addressable, driven by ucm_delta_plan_rows' output with no host
 * round trip: for every (layer l, request row, slot j) with
 * sel = load_sel[l][row][j] >= 0, the K and V slices of stored block
 * src_table[row][sel] are copied into cache block dst_table[row][j] of layer l.
 *   layers      dev array of n_layers cache pointers (as for the other KV moves)
 *   pool        dev: stored blocks of pool_block_bytes each, slice (layer, K|V)
 *               of a block at ((store_first_layer + l)*2 + kv)*block_bytes -
 *               the get_offset layout (esa.py:124-135, tp_size 1);
 *               store_first_layer is the model layer layers[0] belongs to
 *   load_sel    dev int32 [n_layers][table_rows][n_slots] (load_phys of the plan)
 *   src_table   dev int32 [table_rows][src_stride]: pool block holding logical
 *               block i of the request, -1 = not stored (skipped)
 *   dst_table   dev int32 [table_rows][dst_stride]: cache block id of slot j
 *               (the request's first top_k vLLM blocks, esa.py:311); layer l
 *               reads the table dst_layer_stride elements after layer l-1's
 *               (0: one table for all layers)
 *   load_count  dev int32 [n_layers][table_rows] or NULL: only the first
 *               load_count entries of a row of load_sel are followed
 *   rows        dev int32 [batch] or NULL (then request b uses row b)
 * Ids outside the pool or the cache are skipped, never dereferenced.
 */
int ucm_kv_load_planned(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                        int num_blocks, const void* pool, int64_t pool_blocks, size_t pool_block_bytes,
                        int store_first_layer, const int32_t* load_sel, int n_slots,
                        const int32_t* src_table, int src_stride, const int32_t* dst_table,
                        int dst_stride, int64_t dst_layer_stride, const int32_t* load_count,
                        const int32_t* rows, int batch, int table_rows, ucm_stream_t stream);
int ucm_kv_load_planned_tp(void* const* layers, int n_layers, size_t kv_stride, size_t block_bytes,
                           int num_blocks, const void* pool, int64_t pool_blocks, size_t pool_block_bytes,
                           int store_first_layer, const int32_t* load_sel, int n_slots,
                           const int32_t* src_table, int src_stride, const int32_t* dst_table,
                           int dst_stride, int64_t dst_layer_stride, const int32_t* load_count,
                           const int32_t* rows, int batch, int table_rows, int rank, int tp_size,
                           ucm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* UCM_HIP_H */
