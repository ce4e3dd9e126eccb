/*
 * litekv.h -- C ABI of liblitekv.so: the paged-KV-cache attention path of
 * lite_llama, written for one AMD Instinct MI355X (gfx950).
 *
 * Conventions shared by every entry point
 *   - every pointer is a DEVICE pointer, 16-byte aligned, owned by the caller;
 *     the library never allocates, frees or synchronises;
 *   - calls only enqueue work on `stream` (a hipStream_t passed as void*;
 *     NULL is the default stream) and return at once;
 *   - the return value is a status: LITEKV_OK, or non-zero with a message
 *     readable through litekv_last_error() (thread local);
 *   - launch shapes depend only on the host scalars passed in, never on device
 *     data, so a call sequence can be recorded once and replayed;
 *   - data is fp16 ("half"), indices are int32, element strides are in
 *     elements (not bytes) and passed as int64.
 *
 * KV pool layout (one per layer), identical to the reference's
 * `gpu_kv_buffer[l]` (lite_llama/executor/paged_attention.py:54-62):
 *     kv_pool[num_pages * page_size][2 * num_kv_heads][head_dim]  fp16
 * heads [0, Hkv) of a slot are K, heads [Hkv, 2*Hkv) are V
 * (lite_llama/models/qwen3.py:68-69). slot = page_id * page_size + offset
 * (lite_llama/executor/paged_attention.py:141-146, 347-354), so a page is one
 * contiguous run of page_size * 2 * Hkv * head_dim * 2 bytes.
 *
 * Supported shapes: Hq % Hkv == 0, Hq / Hkv <= 64 (the decode kernels hold the
 * query heads of a kv head in the 16 columns of a tile; a larger group runs as
 * slices of up to 16, each reading the head's K/V; the reference's grids are
 * per query head, lite_llama/kernels/flashdecoding.py:44, 170-175); page_size
 * 16, 32, 64, 128 or 256 (the reference's --page_size,
 * lite_llama/server.py:1038-1161, "typically 16-256",
 * lite_llama/executor/paged_attention.py:27): the attention kernels walk a
 * larger page as 2 .. 16 consecutive 16-token pieces; head_dim 128 and 64 on the MFMA-tiled kernels, and 32, 64 or 256
 * (the reference kernels take the head dim as a block size,
 * lite_llama/kernels/flashdecoding.py:305, 393-396) through the same entry
 * points on one general kernel with fp32 arithmetic where no tiled kernel
 * exists (32 and 256): it writes the final rows in a single launch whatever
 * schedule was asked for, and uses no workspace.
 */
#ifndef LITEKV_H
#define LITEKV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LITEKV_OK 0
#define LITEKV_ERR_INVALID_ARGUMENT 1
#define LITEKV_ERR_LAUNCH 2

#define LITEKV_ABI_VERSION 3

/* ABI version of the loaded library (LITEKV_ABI_VERSION at build time). */
int litekv_abi_version(void);

/* Message of the last failing call made by this thread ("" if none). */
const char *litekv_last_error(void);

/*
 * KV append. Replaces `update_kv_buffer(KV_Values, Select_Index, KV_Buffer)`
 * (lite_llama/kernels/update_kv_buffer.py:46-81) together with the
 * `torch.cat([xk, xv], dim=-2)` its callers run first
 * (lite_llama/models/qwen3.py:29, 62):
 *     kv_pool[slot_mapping[t]][0:Hkv]     = k[t]
 *     kv_pool[slot_mapping[t]][Hkv:2*Hkv] = v[t]      for t in [0, num_tokens)
 * k and v are [num_tokens][Hkv][head_dim] with the given token strides (the
 * inner [Hkv][head_dim] block contiguous), so the two halves of an already
 * concatenated [T][2*Hkv][D] tensor can be passed without a copy.
 * A slot outside [0, num_slots) is skipped (padding rows of a replayed batch).
 * The copy is bit exact.
 */
int litekv_kv_append(const void *k, const void *v,
                     int64_t k_token_stride, int64_t v_token_stride,
                     const int32_t *slot_mapping, void *kv_pool,
                     int32_t num_tokens, int32_t num_kv_heads, int32_t head_dim,
                     int64_t num_slots, void *stream);

/*
 * Fused epilogue of the QKV projection, the step before the KV append on the
 * reference's path (Qwen3Attention._get_qkv, lite_llama/models/qwen3.py:109-130,
 * followed by Attention.context_forward / token_forward :29, :62): per-head
 * RMSNorm of q and k (skip_rmsnorm with residual None ->
 * rms_norm_kernel, lite_llama/kernels/skip_rmsnorm.py:117-146), rotary
 * embedding of q and k (rope_emb_forward, lite_llama/kernels/rope_emb.py:6-131;
 * first-half / second-half pairing, the first head_dim/2 entries of each cos /
 * sin row are used), `torch.cat([xk, xv])` and `update_kv_buffer`, in one
 * launch:
 *     q[t][h]                             = rope(norm(q[t][h]) * q_norm_weight)      in place
 *     kv_pool[slot_mapping[t]][h]         = rope(norm(k[t][h]) * k_norm_weight)
 *     kv_pool[slot_mapping[t]][Hkv + h]   = v[t][h]                                   bit exact
 * norm(x) = x / sqrt(mean(x^2) + rms_eps) in fp32, rounded to fp16 before the
 * weight multiply, the product rounded to fp16 (as the reference); the
 * rotation is evaluated in fp32 from those fp16 values and rounded once.
 *   q_norm_weight, k_norm_weight   [head_dim] fp16, or both NULL (models
 *                                  without QK norm: llama.py, qwen2.py)
 *   cos_rows, sin_rows             [num_tokens][cos_sin_token_stride] fp16, the
 *                                  row of each token's position (what
 *                                  RotaryEmbedding.forward returns,
 *                                  RotaryEmbedding.py:183-200), or both NULL
 *   slot outside [0, num_slots)    k / v of that token are not stored; q is
 *                                  still processed
 */
int litekv_qk_norm_rope_append(void *q, int64_t q_token_stride, const void *k,
                               int64_t k_token_stride, const void *v, int64_t v_token_stride,
                               const void *q_norm_weight, const void *k_norm_weight,
                               const void *cos_rows, const void *sin_rows,
                               int64_t cos_sin_token_stride, const int32_t *slot_mapping,
                               void *kv_pool, int32_t num_tokens, int32_t num_q_heads,
                               int32_t num_kv_heads, int32_t head_dim, int64_t num_slots,
                               float rms_eps, void *stream);

/*
 * Page gather / page copy. The reference has no page-move operation (its
 * allocator never moves KV: lite_llama/executor/paged_attention.py:1-11);
 * these serve copy-on-write of a shared page and pool compaction:
 *     dst_pool[page dst_ids[i]] = src_pool[page src_ids[i]]   for i in [0, n)
 * dst_ids == NULL means dst page i. page_bytes must be a multiple of 16.
 * src_pool may equal dst_pool (litekv_page_copy) provided no destination page
 * is also a source page of a different move and destinations are distinct.
 * Ids outside [0, num_src_pages) / [0, num_dst_pages) are skipped. Bit exact.
 */
int litekv_page_gather(const void *src_pool, void *dst_pool,
                       const int32_t *src_ids, const int32_t *dst_ids,
                       int32_t n, int64_t page_bytes,
                       int64_t num_src_pages, int64_t num_dst_pages,
                       void *stream);

int litekv_page_copy(void *kv_pool, const int32_t *src_ids,
                     const int32_t *dst_ids, int32_t n, int64_t page_bytes,
                     int64_t num_pages, void *stream);

/*
 * Paged flash-decoding. Replaces `flash_decoding(q, k_cache, v_cache,
 * qk_scale, b_req_tokens_table, b_seq_len, max_actual_seq_len)`
 * (lite_llama/kernels/flashdecoding.py:294-342; stage 1 :6-138, stage 2
 * :199-267):  out[b][h] = softmax(q[b][h] . K_b[h / (Hq/Hkv)]^T * scale) V_b,
 * over the seq_lens[b] tokens of sequence b, whose token t lives in page
 * block_table[b][t / page_size] at offset t % page_size.
 *
 *   q            [B][Hq][D] fp16, batch stride q_batch_stride, heads contiguous
 *   block_table  [B][block_table_stride] int32 page ids (the per-page
 *                equivalent of the reference's per-token
 *                b_req_tokens_table, paged_attention.py:166-170)
 *   seq_lens     [B] int32, tokens to attend over (already counting the token
 *                appended this step, model_executor.py:893-911); 0 gives zeros
 *   out          [B][Hq][D] fp16, contiguous
 *   max_splits   S >= 1: upper bound of KV splits per sequence = grid extent
 *   min_pages_per_split  sequence b uses
 *                n_b = clamp(ceil(pages_b / min_pages_per_split), 1, S) splits
 *                with page boundaries floor(s * pages_b / n_b): a pure function
 *                of (seq_lens[b], S, min_pages_per_split), so results do not
 *                depend on timing
 *   workspace    litekv_paged_decode_workspace_bytes(B, Hq, D, S) bytes:
 *                fp32 partial outputs [B][Hq][S][D] then natural-log
 *                log-sum-exp [B][Hq][S] (the reference's mid_o /
 *                mid_o_logexpsum, flashdecoding.py:310-321); may be NULL when
 *                S == 1
 *   softmax_scale natural scale (1/sqrt(D)); exp, not exp2, semantics
 * Two launches: split kernel, then the merge in split-index order.
 */
size_t litekv_paged_decode_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                           int32_t head_dim, int32_t max_splits);

int litekv_paged_decode(const void *q, int64_t q_batch_stride,
                        const void *kv_pool, const int32_t *block_table,
                        int32_t block_table_stride, const int32_t *seq_lens,
                        void *out, void *workspace, size_t workspace_bytes,
                        int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                        int32_t head_dim, int32_t page_size, int64_t num_pages,
                        int32_t max_splits, int32_t min_pages_per_split,
                        float softmax_scale, void *stream);

/*
 * The two stages of litekv_paged_decode on their own (same arguments), for
 * callers that time or schedule them separately
 * (flash_decode_stage1 / flash_decode_stage2, flashdecoding.py:141-196,
 * 270-291).
 */
int litekv_paged_decode_split(const void *q, int64_t q_batch_stride,
                              const void *kv_pool, const int32_t *block_table,
                              int32_t block_table_stride, const int32_t *seq_lens,
                              void *out, void *workspace, size_t workspace_bytes,
                              int32_t batch, int32_t num_q_heads,
                              int32_t num_kv_heads, int32_t head_dim,
                              int32_t page_size, int64_t num_pages,
                              int32_t max_splits, int32_t min_pages_per_split,
                              float softmax_scale, void *stream);

int litekv_paged_decode_merge(const int32_t *seq_lens, void *out,
                              const void *workspace, size_t workspace_bytes,
                              int32_t batch, int32_t num_q_heads,
                              int32_t head_dim, int32_t page_size,
                              int32_t max_splits, int32_t min_pages_per_split,
                              void *stream);

/*
 * litekv_paged_decode for callers that cannot allocate device memory. It has
 * no counterpart in the reference (whose flash_decoding allocates mid_o /
 * mid_o_logexpsum with torch.empty on every call, flashdecoding.py:310-321);
 * it is for code under HIP graph capture, serving loops that must not reach an
 * allocator and harnesses that forbid hipMalloc. Same arguments, result and
 * two launches as litekv_paged_decode, minus the workspace: the fp32 partial
 * rows and log-sum-exps live in a device array built into the library,
 * LITEKV_STATIC_SCRATCH_BYTES long, which every GPU the library runs on holds
 * until the process ends. The call itself allocates and frees nothing.
 *   limit   litekv_paged_decode_workspace_bytes(batch, num_q_heads, head_dim,
 *           max_splits) must not exceed LITEKV_STATIC_SCRATCH_BYTES, else
 *           LITEKV_ERR_INVALID_ARGUMENT (32 MiB: e.g. batch 32 x 64 query
 *           heads x 31 splits, or batch 128 x 32 heads x 15 splits)
 *   sharing every call on a GPU uses that GPU's one array: calls that overlap
 *           in time on one GPU (two streams, two threads) race; calls on one
 *           stream are ordered. Nothing in it has to start at zero: the merge
 *           reads only the cells the split launch of the same call wrote.
 *           A host thread that enters while another is still enqueueing its
 *           launches on the same GPU gets LITEKV_ERR_INVALID_ARGUMENT; overlap
 *           on the GPU between streams is the caller's to exclude.
 *   set-up  the array's address on a device is looked up on the first call
 *           made with that device current (no allocation). Any call does it,
 *           also one with batch 0: make that call before capturing a graph. A
 *           first call that finds its stream capturing returns
 *           LITEKV_ERR_INVALID_ARGUMENT and leaves the capture intact.
 */
#define LITEKV_STATIC_SCRATCH_BYTES (32u << 20)

int litekv_paged_decode_static(const void *q, int64_t q_batch_stride, const void *kv_pool,
                               const int32_t *block_table, int32_t block_table_stride,
                               const int32_t *seq_lens, void *out, int32_t batch,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t page_size, int64_t num_pages, int32_t max_splits,
                               int32_t min_pages_per_split, float softmax_scale, void *stream);

/*
 * Paged flash-decoding, balanced schedule. Same
 * result contract as litekv_paged_decode (it replaces the same reference
 * function, lite_llama/kernels/flashdecoding.py:294-342), other work
 * decomposition: the pages of all sequences, concatenated in batch order, are
 * cut into `chunks` equal pieces per kv head; a workgroup of up to 8 wavefronts
 * (one per kv head) streams one piece and crosses sequence boundaries as
 * needed, so the launch is evenly loaded whatever the length distribution. The
 * piece of sequence b inside chunk c is partial slot c + b; a sequence inside a
 * single chunk is written directly; the others are merged in chunk order by a
 * small second launch (the reference's stage 2, flashdecoding.py:242-267).
 *
 * Step plan. The cuts depend only on (block_table, seq_lens, chunks), which
 * are the same for every layer of a decode step (the reference builds its
 * per-step metadata once as well, model_executor.py:893-911), so they are
 * computed once per step by litekv_decode_plan into `plan`
 * (litekv_decode_plan_bytes bytes) and consumed by every layer's launch.
 * Launches sharing a workspace must not overlap in time.
 *
 * Optional fused append. With k_new / v_new non-NULL ([B][Hkv][D], batch
 * strides given) the launch also performs this step's KV append: the rows are
 * written, bit exact, to logical position seq_lens[b] - 1 of sequence b (the
 * slot the reference passes as cur_select_index, paged_attention.py:310-317)
 * and take part in the attention. It replaces
 * the separate update_kv_buffer launch of Attention.token_forward
 * (lite_llama/models/qwen3.py:53-75).
 *
 *   chunks     pieces per kv head (>= 1); litekv_paged_decode_balanced_chunks()
 *              returns the count that gives each CU of the current device one
 *              workgroup
 *   workspace  litekv_paged_decode_balanced_workspace_bytes(B, Hq, D, chunks):
 *              fp32 partials [chunks + B][Hq][D], then log-sum-exp
 *              [chunks + B][Hq]
 *   block_table_stride, chunks  must equal the values the plan was made with
 */
int32_t litekv_paged_decode_balanced_chunks(int32_t num_kv_heads);

/* The chunk count for a step behind `shared_pages` shared pages
 * (litekv_paged_decode_prefix): the workgroups that attend the shared pages and
 * those that stream the private pages are one launch and should all be
 * resident at once, so the private pages get the compute units the others
 * leave. pool_is_fp16: 0 for a pool of 8-bit codes. Falls back to
 * litekv_paged_decode_balanced_chunks for arguments it cannot use. */
int32_t litekv_paged_decode_prefix_chunks(int32_t batch, int32_t num_q_heads,
                                          int32_t num_kv_heads, int32_t head_dim,
                                          int32_t page_size, int32_t shared_pages,
                                          int32_t pool_is_fp16);

size_t litekv_paged_decode_balanced_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                    int32_t head_dim, int32_t chunks);

size_t litekv_decode_plan_bytes(int32_t batch, int32_t block_table_stride,
                                int32_t num_kv_heads, int32_t chunks);
/* The same for a pool whose pages hold page_size (16 .. 256) tokens: the plan
 * lists 16-token pages, page_size / 16 per block-table entry.
 * litekv_decode_plan_bytes is the page_size 16 case. 0 for another page_size. */
size_t litekv_decode_plan_bytes_paged(int32_t batch, int32_t block_table_stride,
                                      int32_t num_kv_heads, int32_t chunks, int32_t page_size);

int litekv_decode_plan(const int32_t *block_table, int32_t block_table_stride,
                       const int32_t *seq_lens, int32_t batch, int32_t num_kv_heads,
                       int32_t page_size, int64_t num_pages, int32_t chunks,
                       void *plan, size_t plan_bytes, void *stream);

int litekv_paged_decode_balanced(const void *q, int64_t q_batch_stride, void *kv_pool,
                                 const int32_t *seq_lens, void *plan, size_t plan_bytes,
                                 const void *k_new, const void *v_new,
                                 int64_t k_new_stride, int64_t v_new_stride,
                                 void *out, void *workspace, size_t workspace_bytes,
                                 int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                 int32_t head_dim, int32_t page_size, int64_t num_pages,
                                 int32_t block_table_stride, int32_t chunks,
                                 float softmax_scale, void *stream);

/*
 * Balanced paged decode for a batch whose sequences all start with the same
 * `shared_pages` physical pages (block_table[b][0 .. shared_pages) identical
 * for every b): a cached system prompt or few-shot prefix, which the
 * reference maps into every request's table by reference
 * (ModelExecutor.share_paged_prefix_from_cache, model_executor.py:570-620;
 * PagedReqTokensManager.share_req_from_pages, paged_attention.py:252-274) and
 * then reads once per sequence and query head (flashdecoding.py:84-94). Here
 * the shared pages are attended once for the whole batch: the (sequence, query
 * head) pairs of one kv head form the columns of an MFMA-tiled kernel over the
 * prefix keys, whose partial rows join the log-sum-exp merge of the private
 * pages. Result contract as litekv_paged_decode_balanced (same tolerance; not
 * bit-identical to it, the summation order differs).
 *
 *   litekv_decode_plan_prefix   as litekv_decode_plan, over the pages after
 *                the first shared_pages of every sequence
 *   shared_pages must equal the value the plan was made with; 0 gives
 *                litekv_paged_decode_balanced. Every sequence with
 *                seq_lens[b] > 0 must hold at least shared_pages full pages.
 *   block_table  [B][block_table_stride]; only row 0's first shared_pages
 *                entries are read by this call (the rest is in the plan)
 *   workspace    litekv_paged_decode_prefix_workspace_bytes(B, Hq, D, chunks)
 */
size_t litekv_paged_decode_prefix_workspace_bytes(int32_t batch, int32_t num_q_heads,
                                                  int32_t head_dim, int32_t chunks);

int litekv_decode_plan_prefix(const int32_t *block_table, int32_t block_table_stride,
                              const int32_t *seq_lens, int32_t batch, int32_t num_kv_heads,
                              int32_t page_size, int64_t num_pages, int32_t chunks,
                              int32_t shared_pages, void *plan, size_t plan_bytes, void *stream);

int litekv_paged_decode_prefix(const void *q, int64_t q_batch_stride, void *kv_pool,
                               const int32_t *block_table, const int32_t *seq_lens, void *plan,
                               size_t plan_bytes, const void *k_new, const void *v_new,
                               int64_t k_new_stride, int64_t v_new_stride, void *out,
                               void *workspace, size_t workspace_bytes, int32_t batch,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t page_size, int64_t num_pages, int32_t block_table_stride,
                               int32_t chunks, int32_t shared_pages, float softmax_scale,
                               void *stream);

/*
 * FP8 KV pool (no counterpart in the reference: its README lists FP8 as "not
 * yet stabilized", README.md:89, and its only low-precision KV code is the
 * unused int8 prefill kernel lite_llama/kernels/others/
 * context_flashattention_nopad.py:374-553; the layout and call shape follow
 * the fp16 entry points above). The pool is
 *     kv_pool_fp8[num_pages * page_size][2 * num_kv_heads][head_dim]  bytes
 * of OCP E4M3FN codes (bias 7, largest finite value 448, no infinities), K
 * heads then V heads, with one fp32 scale per head, scales[2 * num_kv_heads]
 * (K heads, then V heads):
 *     code  = e4m3(clamp(x * (1 / scale), -448, 448)), round to nearest even
 *     value = decode(code) * scale
 * A page is one contiguous run of page_size * 2 * Hkv * head_dim bytes, so
 * litekv_page_copy / litekv_page_gather move fp8 pages as they are.
 *
 * litekv_kv_append_fp8: litekv_kv_append into an fp8 pool (k, v fp16 rows).
 * The stored codes are a pure function of the row and the scale.
 *
 * litekv_page_dequant: dst_pool[page dst_ids[i]] = fp16(value) of page
 * src_ids[i], for the prefill entry points, which read fp16 pools (a chunk
 * that attends to cached fp8 history first turns the pages it needs into a
 * scratch fp16 pool). dst_ids NULL means page i; ids out of range are skipped.
 *
 * litekv_paged_decode_balanced_fp8: litekv_paged_decode_balanced over an fp8
 * pool, same plan, workspace and result contract. Decoding E4M3 to fp16 is
 * exact, so the result is fp16 attention over the decoded values: the K scale
 * joins the softmax scale, the V scale the final normalisation. k_new / v_new
 * (fp16) are quantised as by litekv_kv_append_fp8 and attended as stored.
 */
int litekv_kv_append_fp8(const void *k, const void *v, int64_t k_token_stride,
                         int64_t v_token_stride, const int32_t *slot_mapping,
                         void *kv_pool_fp8, const float *scales, int32_t num_tokens,
                         int32_t num_kv_heads, int32_t head_dim, int64_t num_slots,
                         void *stream);

/* litekv_qk_norm_rope_append into an fp8 pool: the rotated k row and the v row are quantised as
 * by litekv_kv_append_fp8 (same codes for the same fp16 row); q as in the fp16 variant. */
int litekv_qk_norm_rope_append_fp8(void *q, int64_t q_token_stride, const void *k,
                                   int64_t k_token_stride, const void *v, int64_t v_token_stride,
                                   const void *q_norm_weight, const void *k_norm_weight,
                                   const void *cos_rows, const void *sin_rows,
                                   int64_t cos_sin_token_stride, const int32_t *slot_mapping,
                                   void *kv_pool_fp8, const float *scales, int32_t num_tokens,
                                   int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                   int64_t num_slots, float rms_eps, void *stream);

int litekv_page_dequant(const void *kv_pool_fp8, void *dst_pool, const int32_t *src_ids,
                        const int32_t *dst_ids, int32_t n, const float *scales,
                        int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                        int64_t num_src_pages, int64_t num_dst_pages, void *stream);

int litekv_paged_decode_balanced_fp8(const void *q, int64_t q_batch_stride, void *kv_pool_fp8,
                                     const float *scales, const int32_t *seq_lens, void *plan,
                                     size_t plan_bytes, const void *k_new, const void *v_new,
                                     int64_t k_new_stride, int64_t v_new_stride, void *out,
                                     void *workspace, size_t workspace_bytes, int32_t batch,
                                     int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                     int32_t page_size, int64_t num_pages,
                                     int32_t block_table_stride, int32_t chunks,
                                     float softmax_scale, void *stream);

/*
 * litekv_paged_decode (per-sequence splits, both stages) over an fp8 pool; the
 * merge stage is litekv_paged_decode_merge, which never touches the pool.
 */
int litekv_paged_decode_fp8(const void *q, int64_t q_batch_stride, const void *kv_pool_fp8,
                            const float *scales, const int32_t *block_table,
                            int32_t block_table_stride, const int32_t *seq_lens, void *out,
                            void *workspace, size_t workspace_bytes, int32_t batch,
                            int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t page_size, int64_t num_pages, int32_t max_splits,
                            int32_t min_pages_per_split, float softmax_scale, void *stream);

/*
 * litekv_paged_decode with the step's append fused in: the wavefront that
 * attends a sequence's last page first writes the step's token (rows k_new[b],
 * v_new[b] of [batch][num_kv_heads][128] fp16, element strides per sequence)
 * at logical position seq_lens[b] - 1 of the pages the block table names, as
 * litekv_kv_append would through that token's slot, and attends it. Replaces,
 * in one launch for max_splits == 1, the reference's per-layer pair
 * update_kv_buffer + flash_decoding (models/qwen3.py:62-74;
 * kernels/update_kv_buffer.py:46-81, kernels/flashdecoding.py:294-342) for
 * steps small enough that one wavefront per (sequence, kv head) beats the
 * balanced cut. The _fp8 variant quantises the rows with the pool's scales
 * exactly as litekv_kv_append_fp8 does.
 */
int litekv_paged_decode_append(const void *q, int64_t q_batch_stride, void *kv_pool,
                               const int32_t *block_table, int32_t block_table_stride,
                               const int32_t *seq_lens, const void *k_new, const void *v_new,
                               int64_t k_new_stride, int64_t v_new_stride, void *out,
                               void *workspace, size_t workspace_bytes, int32_t batch,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t page_size, int64_t num_pages, int32_t max_splits,
                               int32_t min_pages_per_split, float softmax_scale, void *stream);
int litekv_paged_decode_append_fp8(const void *q, int64_t q_batch_stride, void *kv_pool_fp8,
                                   const float *scales, const int32_t *block_table,
                                   int32_t block_table_stride, const int32_t *seq_lens,
                                   const void *k_new, const void *v_new, int64_t k_new_stride,
                                   int64_t v_new_stride, void *out, void *workspace,
                                   size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                   int64_t num_pages, int32_t max_splits,
                                   int32_t min_pages_per_split, float softmax_scale, void *stream);

/*
 * litekv_paged_decode_prefix over an fp8 pool (plan from
 * litekv_decode_plan_prefix, workspace from
 * litekv_paged_decode_prefix_workspace_bytes): the shared pages of a cached
 * prefix, which the reference maps into every request by reference
 * (lite_llama/executor/model_executor.py:570-620), are attended once for the
 * batch from their codes.
 */
int litekv_paged_decode_prefix_fp8(const void *q, int64_t q_batch_stride, void *kv_pool_fp8,
                                   const float *scales, const int32_t *block_table,
                                   const int32_t *seq_lens, void *plan, size_t plan_bytes,
                                   const void *k_new, const void *v_new, int64_t k_new_stride,
                                   int64_t v_new_stride, void *out, void *workspace,
                                   size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                   int64_t num_pages, int32_t block_table_stride, int32_t chunks,
                                   int32_t shared_pages, float softmax_scale, void *stream);

/*
 * Advances the metadata of a decode batch by one token on the device, so that
 * a captured graph of a decode step replays without host work. Replaces, per
 * step, PagedReqTokensManager.extend_req + batch_metadata
 * (lite_llama/executor/paged_attention.py:287-359), update_kv_index
 * (lite_llama/kernels/update_kv_index.py:41-74) and the host-to-device copies
 * of cur_select_index / b_seq_len / b_req_idx in NpuGraphRunner.replay
 * (lite_llama/executor/npu_graph.py:183-197). Pages must have been reserved
 * ahead by the host (ensure_req_capacity, paged_attention.py:222-250): the
 * kernel only reads page lists.
 *
 *   request_tables [max_requests][request_table_stride] int32: the page list
 *                  of every request slot (the executor's device block table)
 *   request_ids    [B] int32: request slot of each batch row
 *   capacity       [B] int32 or NULL: tokens each row may grow to (its
 *                  reserved pages * page_size); NULL: width * page_size
 *   seq_lens       [B] int32, in/out: += increment (0 recomputes the outputs
 *                  for the lengths as they are, 1 is a decode step)
 *   seq_lens_i64   [B] int64 or NULL: copy of seq_lens (b_seq_len)
 *   slot_mapping   [B] int32 out: slot of logical token seq_lens[b] - 1
 *                  (cur_select_index); -1 when the row is empty or refused
 *   position_ids   [B] int64 or NULL: seq_lens[b] - 1 (0 for an empty or
 *                  refused row)
 *   block_table    [B][block_table_stride] int32 out: first `width` entries
 *                  of each row's page list, in batch order
 *   overflow       int32[1] or NULL: set to 1 (never cleared here) when a row
 *                  was refused (bad request id, negative length, capacity
 *                  reached). A refused row gets length -1 and slot -1 and
 *                  stays refused on later steps: the decode and append
 *                  kernels treat it as empty (zero output, nothing stored),
 *                  so no cached token is overwritten; the caller reads the
 *                  flag at its next synchronisation and rebuilds the batch
 */
int litekv_decode_advance(const int32_t *request_tables, int64_t request_table_stride,
                          int32_t max_requests, const int32_t *request_ids,
                          const int32_t *capacity, int32_t *seq_lens, int64_t *seq_lens_i64,
                          int32_t *slot_mapping, int64_t *position_ids, int32_t *block_table,
                          int64_t block_table_stride, int32_t width, int32_t *overflow,
                          int32_t batch, int32_t page_size, int64_t num_pages,
                          int32_t increment, void *stream);

/*
 * Varlen causal prefill over paged KV. Replaces
 * `paged_chunk_flash_attention(q, k_cache, v_cache, sm_scale, req_token_table,
 * req_ids, q_start_loc, context_lens, q_seq_lens, max_q_len)`
 * (lite_llama/kernels/paged_chunk_flashattention.py:225-327, kernel :58-176):
 * query row m of sequence b sits at logical position context_lens[b] + m and
 * attends to keys 0 .. context_lens[b] + m read through block_table[b].
 * With context_lens == NULL (all zero) it is the paged form of
 * `flash_attention2_no_pad` (lite_llama/kernels/flashattention2_nopad.py:169-221).
 *
 *   q, out        [T][Hq][D] fp16 packed rows, token strides given
 *   cu_q_lens     [B+1] int32, rows of sequence b are
 *                 [cu_q_lens[b], cu_q_lens[b+1])
 *   context_lens  [B] int32 or NULL
 *   max_q_len     host upper bound of the per-sequence query length (grid)
 *   softmax_scale natural scale; callers holding the reference's
 *                 log2(e)-folded scale (lite_llama/models/qwen3.py:295-298)
 *                 divide it out first
 */
int litekv_paged_prefill(const void *q, int64_t q_token_stride,
                         const void *kv_pool, const int32_t *block_table,
                         int32_t block_table_stride, const int32_t *cu_q_lens,
                         const int32_t *context_lens, void *out,
                         int64_t out_token_stride, int32_t batch,
                         int32_t num_q_heads, int32_t num_kv_heads,
                         int32_t head_dim, int32_t page_size, int64_t num_pages,
                         int32_t max_q_len, float softmax_scale, void *stream);

/*
 * The same for launches with too few query rows to fill the device: one
 * request's chunk over a long history, the case of the reference's chunked
 * prefill (`prefill_chunk_size`, lite_llama/continuous_batching.py:194-611
 * calls paged_chunk_flash_attention once per chunk). Every block of query rows
 * is cut along its keys into `key_slices` runs of key tiles, one workgroup
 * each; the slices leave fp32 partial rows + log-sum-exps in `workspace`, and
 * a second launch folds them in slice order (results do not depend on timing;
 * they differ from litekv_paged_prefill's within fp32 rounding of the merge).
 * head_dim 64 or 128, 2 <= key_slices <= 8.
 *
 *   litekv_paged_prefill_key_slices  the count with the smallest estimated
 *       time when the longest row sees max_kv_len keys (history + chunk):
 *       key tiles per workgroup at the rate its share of a compute unit
 *       gives, against a merge launch and a partial row per query row, head
 *       and slice; 1: do not split (call litekv_paged_prefill) -- launches
 *       that fill the device, short histories, fresh prompts
 *   num_tokens    T, the query rows of the launch (= cu_q_lens[batch])
 *   workspace     litekv_paged_prefill_split_workspace_bytes(T, Hq, D,
 *                 key_slices) bytes, 16-byte aligned; launches that share it
 *                 must be ordered on one stream
 */
size_t litekv_paged_prefill_split_workspace_bytes(int64_t num_tokens,
                                                  int32_t num_q_heads,
                                                  int32_t head_dim,
                                                  int32_t key_slices);
int32_t litekv_paged_prefill_key_slices(int32_t batch, int32_t num_q_heads,
                                        int32_t num_kv_heads, int32_t head_dim,
                                        int32_t max_q_len, int64_t max_kv_len);
int litekv_paged_prefill_split(const void *q, int64_t q_token_stride,
                               const void *kv_pool, const int32_t *block_table,
                               int32_t block_table_stride,
                               const int32_t *cu_q_lens,
                               const int32_t *context_lens, void *out,
                               int64_t out_token_stride, int32_t batch,
                               int32_t num_q_heads, int32_t num_kv_heads,
                               int32_t head_dim, int32_t page_size,
                               int64_t num_pages, int32_t max_q_len,
                               int64_t num_tokens, int32_t key_slices,
                               void *workspace, size_t workspace_bytes,
                               float softmax_scale, void *stream);

/* litekv_paged_prefill_split over a pool of 8-bit codes with per-head scales
 * (fp8 E4M3, or int8 when pool_is_int8 is not 0): see litekv_paged_prefill_fp8
 * / _int8 below for the pool, litekv_paged_prefill_split for the rest. */
int litekv_paged_prefill_split_q8(const void *q, int64_t q_token_stride,
                                  const void *kv_pool, const float *kv_scales,
                                  int32_t pool_is_int8,
                                  const int32_t *block_table,
                                  int32_t block_table_stride,
                                  const int32_t *cu_q_lens,
                                  const int32_t *context_lens, void *out,
                                  int64_t out_token_stride, int32_t batch,
                                  int32_t num_q_heads, int32_t num_kv_heads,
                                  int32_t head_dim, int32_t page_size,
                                  int64_t num_pages, int32_t max_q_len,
                                  int64_t num_tokens, int32_t key_slices,
                                  void *workspace, size_t workspace_bytes,
                                  float softmax_scale, void *stream);

/*
 * litekv_paged_prefill over an fp8 (E4M3) pool with per-head scales (kv_scales: float32
 * [2 * Hkv], K heads then V heads, value = code * scale), as written by
 * litekv_kv_append_fp8: the chunk rows of a chunked prefill or of a
 * prefix-cache hit attend to their history without the pages being
 * dequantised first (the reference has no counterpart; its paged chunk kernel,
 * lite_llama/kernels/paged_chunk_flashattention.py:225-327, reads fp16 only).
 * The codes are converted exactly; the K scale is applied to the scores and
 * the V scale to the normalised output in fp32.
 */
int litekv_paged_prefill_fp8(const void *q, int64_t q_token_stride,
                             const void *kv_pool, const float *kv_scales,
                             const int32_t *block_table,
                             int32_t block_table_stride,
                             const int32_t *cu_q_lens,
                             const int32_t *context_lens, void *out,
                             int64_t out_token_stride, int32_t batch,
                             int32_t num_q_heads, int32_t num_kv_heads,
                             int32_t head_dim, int32_t page_size,
                             int64_t num_pages, int32_t max_q_len,
                             float softmax_scale, void *stream);

/*
 * Varlen causal prefill over packed contiguous K/V. Replaces
 * `flash_attention2_no_pad(q, k, v, sm_scale, b_start_loc, b_seq_len,
 * max_seq_len)` (lite_llama/kernels/flashattention2_nopad.py:169-221) for
 * callers that hold the fresh K/V rows rather than pages
 * (lite_llama/models/qwen3.py:47-50).
 *   q, out [T][Hq][D]; k, v [T][Hkv][D]; seq_starts, seq_lens [B] int32
 */
int litekv_varlen_prefill(const void *q, int64_t q_token_stride,
                          const void *k, int64_t k_token_stride,
                          const void *v, int64_t v_token_stride,
                          const int32_t *seq_starts, const int32_t *seq_lens,
                          void *out, int64_t out_token_stride, int32_t batch,
                          int32_t num_q_heads, int32_t num_kv_heads,
                          int32_t head_dim, int32_t max_seq_len,
                          int64_t num_tokens, float softmax_scale, void *stream);


/*
 * int8 KV pools. The same pools, scales, call shapes and result contracts as
 * the fp8 entry points above, with signed 8-bit codes instead of E4M3:
 *     code  = clamp(round_to_nearest_even(x * (1 / scale)), -127, 127)
 *     value = code * scale
 * (the reference's int8 cache, lite_llama/kernels/others/
 * context_flashattention_nopad.py:374-553, is read there without scales; the
 * per-head scales are the fp8 pools'). Every code is an fp16 number, so
 * attention over an int8 pool is fp16 attention over the codes with the K
 * scale joining the softmax scale and the V scale the final normalisation.
 * Each function below is its _fp8 namesake (litekv_page_dequant_int8:
 * litekv_page_dequant) for an int8 pool; litekv_page_copy / litekv_page_gather
 * move int8 pages as they are.
 */
int litekv_kv_append_int8(const void *k, const void *v, int64_t k_token_stride,
                         int64_t v_token_stride, const int32_t *slot_mapping,
                         void *kv_pool_int8, const float *scales, int32_t num_tokens,
                         int32_t num_kv_heads, int32_t head_dim, int64_t num_slots,
                         void *stream);

int litekv_qk_norm_rope_append_int8(void *q, int64_t q_token_stride, const void *k,
                                   int64_t k_token_stride, const void *v, int64_t v_token_stride,
                                   const void *q_norm_weight, const void *k_norm_weight,
                                   const void *cos_rows, const void *sin_rows,
                                   int64_t cos_sin_token_stride, const int32_t *slot_mapping,
                                   void *kv_pool_int8, const float *scales, int32_t num_tokens,
                                   int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                   int64_t num_slots, float rms_eps, void *stream);

int litekv_page_dequant_int8(const void *kv_pool_int8, void *dst_pool, const int32_t *src_ids,
                        const int32_t *dst_ids, int32_t n, const float *scales,
                        int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                        int64_t num_src_pages, int64_t num_dst_pages, void *stream);

int litekv_paged_decode_balanced_int8(const void *q, int64_t q_batch_stride, void *kv_pool_int8,
                                     const float *scales, const int32_t *seq_lens, void *plan,
                                     size_t plan_bytes, const void *k_new, const void *v_new,
                                     int64_t k_new_stride, int64_t v_new_stride, void *out,
                                     void *workspace, size_t workspace_bytes, int32_t batch,
                                     int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                     int32_t page_size, int64_t num_pages,
                                     int32_t block_table_stride, int32_t chunks,
                                     float softmax_scale, void *stream);

int litekv_paged_decode_int8(const void *q, int64_t q_batch_stride, const void *kv_pool_int8,
                            const float *scales, const int32_t *block_table,
                            int32_t block_table_stride, const int32_t *seq_lens, void *out,
                            void *workspace, size_t workspace_bytes, int32_t batch,
                            int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t page_size, int64_t num_pages, int32_t max_splits,
                            int32_t min_pages_per_split, float softmax_scale, void *stream);

int litekv_paged_decode_append_int8(const void *q, int64_t q_batch_stride, void *kv_pool_int8,
                                   const float *scales, const int32_t *block_table,
                                   int32_t block_table_stride, const int32_t *seq_lens,
                                   const void *k_new, const void *v_new, int64_t k_new_stride,
                                   int64_t v_new_stride, void *out, void *workspace,
                                   size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                   int64_t num_pages, int32_t max_splits,
                                   int32_t min_pages_per_split, float softmax_scale, void *stream);

int litekv_paged_decode_prefix_int8(const void *q, int64_t q_batch_stride, void *kv_pool_int8,
                                   const float *scales, const int32_t *block_table,
                                   const int32_t *seq_lens, void *plan, size_t plan_bytes,
                                   const void *k_new, const void *v_new, int64_t k_new_stride,
                                   int64_t v_new_stride, void *out, void *workspace,
                                   size_t workspace_bytes, int32_t batch, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int32_t page_size,
                                   int64_t num_pages, int32_t block_table_stride, int32_t chunks,
                                   int32_t shared_pages, float softmax_scale, void *stream);

int litekv_paged_prefill_int8(const void *q, int64_t q_token_stride,
                             const void *kv_pool, const float *kv_scales,
                             const int32_t *block_table,
                             int32_t block_table_stride,
                             const int32_t *cu_q_lens,
                             const int32_t *context_lens, void *out,
                             int64_t out_token_stride, int32_t batch,
                             int32_t num_q_heads, int32_t num_kv_heads,
                             int32_t head_dim, int32_t page_size,
                             int64_t num_pages, int32_t max_q_len,
                             float softmax_scale, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LITEKV_H */
