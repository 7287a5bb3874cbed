/*
 * omnikv_hip.h - C ABI of libomnikv_hip.so: MI355X (gfx950) kernels for OmniKV's
 * dynamic-context-selection decode path.
 *
 * The reference has no FFI layer of its own: the interface it exposes for this
 * path is torch-level Python (modeling/omnikv.py, modeling/spec_cache.py) and,
 * on its serving stack, Triton launchers.  Every entry point below names the
 * reference code whose device work it replaces.  The Python package binds these
 * with ctypes and re-creates the reference's Python signatures on top.
 *
 * Conventions
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer unless its
 *     name starts with host_;
 *   - every call is asynchronous on `stream` (a hipStream_t) and allocates
 *     nothing: scratch comes from the caller as (ws, ws_bytes), sized by
 *     okv_workspace_bytes();
 *   - return value: 0 on success, a negative okv_status otherwise; the library
 *     never throws and never aborts; okv_strerror() names a code and
 *     okv_last_error() gives the detail of the calling thread's last failure;
 *   - calls on different streams, from one or several host threads, may run concurrently
 *     if their workspaces differ (okv_set_option is the exception, see there).
 *
 * Tensors
 *   q, out     (batch, num_q_heads, head_dim) contiguous, same dtype as K/V
 *   K, V       described by okv_kv_layout_t: element (b, t, g, d) of request b,
 *              token t, kv head g lives at
 *                contiguous: base + b*batch_stride + t*token_stride + g*head_stride + d
 *                paged:      base + page_table[b*page_table_stride + t/page_size]*page_stride
 *                                 + (t%page_size)*token_stride + g*head_stride + d
 *              Both the reference's (b, Hkv, N, D) tensors (token_stride = D,
 *              head_stride = N*D) and token-major (N, Hkv, D) storage
 *              (token_stride = Hkv*D, head_stride = D) are expressible; strides
 *              are in elements and must be multiples of 8; bases 16-byte aligned.
 *   scores     (batch, score_stride) float32
 *   idx        (batch, idx_stride) int32, ascending per request
 */
#ifndef OMNIKV_HIP_H
#define OMNIKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* okv_stream_t; /* hipStream_t */

enum okv_status {
  OKV_OK = 0,
  OKV_ERR_INVALID = -1,     /* bad argument (null pointer, misaligned, out of range) */
  OKV_ERR_UNSUPPORTED = -2, /* geometry or dtype the kernels are not built for */
  OKV_ERR_WORKSPACE = -3,   /* ws_bytes smaller than okv_workspace_bytes() */
  OKV_ERR_HIP = -4          /* a HIP runtime call failed */
};

enum okv_dtype { OKV_F32 = 0, OKV_BF16 = 1, OKV_F16 = 2 };

/* How the per-head logits of a token become one score. */
enum okv_head_reduce { OKV_REDUCE_MAX = 0, OKV_REDUCE_SUM = 1 };
enum okv_normalise { OKV_NORM_RAW = 0, OKV_NORM_SOFTMAX = 1 };

enum okv_op {
  OKV_OP_SCORE = 0,
  OKV_OP_TOPK = 1,
  OKV_OP_DENSE_ATTN = 2, /* with or without the fused score output */
  OKV_OP_SPARSE_ATTN = 3,
  OKV_OP_SCORE_WINDOW = 4,
  OKV_OP_DENSE_ATTN_SELECT = 5,
  OKV_OP_DENSE_ATTN_WINDOW = 6
};

typedef struct okv_kv_layout {
  int32_t dtype; /* okv_dtype */
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;
  int64_t token_stride;
  int64_t head_stride;
  int64_t batch_stride;      /* contiguous mode only */
  const int32_t* page_table; /* device; NULL selects contiguous mode */
  int32_t page_size;
  int32_t page_table_stride; /* entries per request */
  int64_t page_stride;
} okv_kv_layout_t;

/* Sizes that determine a workspace: fill what the op uses, zero the rest. */
typedef struct okv_shape {
  int32_t batch;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t max_seq_len;  /* longest scored / attended main segment */
  int32_t max_tail_len; /* sparse attention only */
  int32_t with_scores;  /* dense attention: 1 when the score output is wanted */
} okv_shape_t;

const char* okv_strerror(int status);
const char* okv_last_error(void);
int okv_version(void);

/* Process-wide tuning switches, for A/B measurements.  "attn_variant": 0 (default)
 * runs 16-bit attention / scoring on the matrix-core kernel, 1 forces the portable
 * VALU kernel for every dtype.  "split_rows": rows per split of the attention /
 * scoring pass (a multiple of 16), 0 = automatic.  An option applies to every later
 * call of every thread and changes workspace sizes: set options before sizing
 * workspaces and before other threads call into the library, not while they do.
 * No reference counterpart. */
int okv_set_option(const char* name, int value);

/* Bytes of scratch `op` needs for `shape`.  No reference counterpart: the
 * reference lets torch allocate (alloc_tensor_func in
 * omnikv-lightllm/.../triton_kernel/flash_decoding.py:45-60). */
int okv_workspace_bytes(int op, const okv_shape_t* shape, size_t* out_bytes);

/*
 * Filter-layer scoring.  For each request b and token t < score_len:
 *   logit[h][t] = scale * <q[b][h], K[b][t][h / group]>
 *   RAW:      s[h][t] = logit[h][t]
 *   SOFTMAX:  s[h][t] = softmax over t in [0, score_len) of logit[h][.]
 *   scores[b][t] = max_h or sum_h of s[h][t]
 * Replaces the matmul / softmax / max chain of select_tokens_by_attn_universal,
 * branches `last` (RAW+MAX) and `softmax_before_last` (SOFTMAX+MAX):
 * modeling/omnikv.py:37-58; and the raw-score side output of
 * _fwd_kernel_flash_decode_stage1_with_score + attn_score.max(dim=1):
 * omnikv-lightllm/.../flash_decoding_stage1.py:198-207, flash_decoding.py:76.
 * score_lens: device int32[batch] or NULL (then every request has max_score_len).
 */
int okv_score(const void* q, const void* k_base, const okv_kv_layout_t* layout,
              const int32_t* score_lens, int32_t max_score_len, int32_t batch,
              int32_t head_reduce, int32_t normalise, float scale, float* scores,
              int64_t score_stride, void* ws, size_t ws_bytes, okv_stream_t stream);

/*
 * Window selectors.  q holds the last `window` query positions of every q head
 * (element (b, h, w, d) at q + b*q_batch_stride + h*q_head_stride + w*q_pos_stride + d,
 * strides in elements, multiples of 8; position 0 is the oldest).  For each request b
 * and token t < score_len:
 *   m[w][t]   = max_h softmax over t of (scale * <q[b][h][w], K[b][t][h / group]>)
 *   uniform (exp_decay = 0):  scores[b][t] = ((m[0] + m[1]) + m[2]) + ...
 *   exp     (exp_decay = 1):  scores[b][t] = ((m[0]/2 + m[1])/2 + m[2]) ...
 * i.e. the additions in the order of the loops they replace:
 * select_tokens_by_attn_universal, branches `uniform` and `exp`,
 * modeling/omnikv.py:59-103.  K is read twice in total, not `window` times.
 * 16-bit contiguous K, at most 8 kv heads, group of 1, 2, 4 or 8, window * group <= 64; anything else
 * returns OKV_ERR_UNSUPPORTED (callers then score position by position with
 * okv_score).  Workspace: okv_workspace_bytes(OKV_OP_SCORE_WINDOW, ...).
 */
int okv_score_window(const void* q, int64_t q_batch_stride, int64_t q_head_stride,
                     int64_t q_pos_stride, int32_t window, int32_t exp_decay, const void* k_base,
                     const okv_kv_layout_t* layout, const int32_t* score_lens,
                     int32_t max_score_len, int32_t batch, float scale, float* scores,
                     int64_t score_stride, void* ws, size_t ws_bytes, okv_stream_t stream);

/*
 * A filter layer with a window selector in two passes over K instead of three: the dense
 * attention of okv_dense_attn (q: the current position's query, (batch, num_q_heads, head_dim))
 * and the window scores of okv_score_window (q_window, window, exp_decay: as there; its last
 * position is the current one) over the first score_len tokens.  The attention's pass over K
 * and V also computes every window column's log-sum-exp, which is the first of
 * okv_score_window's two passes; the second follows.  out and scores as from the two calls
 * (scores to rounding: the partial sums are grouped by the attention's splits).
 * score_lens[b] must not exceed seq_lens[b].  Same restrictions as okv_score_window.
 * Replaces, for the selectors `uniform` and `exp`, select_tokens_by_attn_universal
 * (modeling/omnikv.py:59-103, called at :189-198) and the attention of the same layer at
 * :219-227.  Workspace: okv_workspace_bytes(OKV_OP_DENSE_ATTN_WINDOW, ...).
 */
int okv_dense_attn_window(const void* q, const void* q_window, int64_t q_batch_stride,
                          int64_t q_head_stride, int64_t q_pos_stride, int32_t window,
                          int32_t exp_decay, const void* k_base, const void* v_base,
                          const okv_kv_layout_t* layout, const int32_t* seq_lens,
                          int32_t max_seq_len, int32_t batch, float scale, void* out,
                          const int32_t* score_lens, int32_t max_score_len, float* scores,
                          int64_t score_stride, void* ws, size_t ws_bytes, okv_stream_t stream);

/*
 * Per-request top-k of fp32 scores.  Writes the k_b = min(k_per_seg[b], len_b)
 * selected token indices in ASCENDING order.  The selected set holds every value
 * greater than the k-th largest and, among values equal to it, those with the
 * lowest indices.  -0.0 equals +0.0; NaN ranks above +inf.
 * Replaces torch.topk(sorted=True) followed by torch.sort(idx):
 * modeling/omnikv.py:47-48,109; and torch.topk in
 * omnikv-lightllm/.../flash_decoding.py:80-83.
 * seq_lens / k_per_seg: device int32[batch] or NULL (then max_seq_len / max_k
 * apply to every request).  idx_out rows beyond k_b are left untouched.
 * ws may be NULL: then one workgroup per request does all the work.  With a
 * workspace of okv_workspace_bytes(OKV_OP_TOPK) bytes, vectors of 14336 scores or
 * more are processed by many workgroups in chunked passes (the workspace needs no
 * preparation).
 */
int okv_topk(const float* scores, int64_t score_stride, const int32_t* seq_lens,
             int32_t max_seq_len, const int32_t* k_per_seg, int32_t max_k,
             int32_t batch, int32_t* idx_out, int64_t idx_stride, void* ws,
             size_t ws_bytes, okv_stream_t stream);

/*
 * Dense GQA decode attention over all seq_len cached tokens of each request:
 * out[b][h] = softmax_t(scale * <q[b][h], K[b][t][h/group]>) . V[b][.][h/group].
 * When `scores` is not NULL the same pass over K also emits the filter-layer
 * scores of the first score_len tokens, exactly as okv_score would (the softmax
 * of the score is over [0, score_len), that of the attention over [0, seq_len)).
 * Replaces the attention the reference runs on a full layer after
 * OmniKVMultiStageCache.update returns the whole cache
 * (modeling/spec_cache.py:358-369, called from modeling/omnikv.py:219-227) and
 * flash_decode_stage1(_with_score) + flash_decode_stage2
 * (omnikv-lightllm/.../flash_decoding.py:62-75,107-112).
 */
int okv_dense_attn(const void* q, const void* k_base, const void* v_base,
                   const okv_kv_layout_t* layout, const int32_t* seq_lens,
                   int32_t max_seq_len, int32_t batch, float scale, void* out,
                   const int32_t* score_lens, int32_t max_score_len,
                   int32_t head_reduce, int32_t normalise, float* scores,
                   int64_t score_stride, void* ws, size_t ws_bytes,
                   okv_stream_t stream);

/*
 * The whole filter layer in one call: okv_dense_attn with the score output, followed by
 * okv_topk over those scores (seq_lens = score_lens, max_seq_len = max_score_len), with the
 * same results as the two calls: out, scores and idx_out are all written, from one workspace.
 * Replaces the filter layer's selection and the attention that follows it in the same
 * decoder-layer forward: modeling/omnikv.py:173-216 (select_tokens_by_attn_universal, :8-110,
 * called at :189-198) and the attention at :219-227; and flash_decode_stage1_with_score +
 * torch.topk, omnikv-lightllm/.../flash_decoding.py:62-83.
 * Workspace: okv_workspace_bytes(OKV_OP_DENSE_ATTN_SELECT, ...).
 */
int okv_dense_attn_select(const void* q, const void* k_base, const void* v_base,
                          const okv_kv_layout_t* layout, const int32_t* seq_lens,
                          int32_t max_seq_len, int32_t batch, float scale, void* out,
                          const int32_t* score_lens, int32_t max_score_len,
                          int32_t head_reduce, int32_t normalise, float* scores,
                          int64_t score_stride, const int32_t* k_per_seg, int32_t max_k,
                          int32_t* idx_out, int64_t idx_stride, void* ws, size_t ws_bytes,
                          okv_stream_t stream);

/*
 * Fused gather + sparse GQA decode attention.  Request b attends to the rows
 *   K/V[b][idx[b][0 .. sel_len_b)]  followed by  tail_K/V[b][0 .. tail_len_b)
 * with one joint softmax.  idx == NULL means rows 0 .. sel_len_b-1 of K/V (an
 * already gathered buffer).  The tail (tokens generated after the prompt) is
 * (batch, tail_len, Hkv, D)-addressed by its own three strides; tail_k may be
 * NULL when max_tail_len == 0.
 * Replaces index_select in set_idx_on_gpu, torch.cat([part, tail]) in update,
 * and the attention over the result: modeling/spec_cache.py:290-306,337-356,
 * modeling/omnikv.py:219-227; and flash_decode_stage1 over
 * req_to_imp_token_indexs: omnikv-lightllm/.../flash_decoding.py:93-105.
 */
int okv_sparse_attn(const void* q, const void* k_base, const void* v_base,
                    const okv_kv_layout_t* layout, const int32_t* idx,
                    int64_t idx_stride, const int32_t* sel_lens, int32_t max_sel_len,
                    const void* tail_k, const void* tail_v, int64_t tail_token_stride,
                    int64_t tail_head_stride, int64_t tail_batch_stride,
                    const int32_t* tail_lens, int32_t max_tail_len, int32_t batch,
                    float scale, void* out, void* ws, size_t ws_bytes,
                    okv_stream_t stream);

/*
 * okv_sparse_attn without a workspace argument and without any allocation, for callers
 * that can do neither: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  No counterpart in the reference.  Same arguments, same kernels and
 * bit-identical output; the per-(q head, split) partial results go to a fixed array inside
 * the library (okv_noalloc_scratch_bytes() = 4 MiB, held once per GPU the library runs on
 * until the process ends).  Shapes whose okv_workspace_bytes(OKV_OP_SPARSE_ATTN, ...)
 * exceed that return OKV_ERR_WORKSPACE (batch 1 fits up to several 100 000 selected rows, batch
 * 16 several 10 000 per request).  The array is looked up once per device on the first
 * call made with that device current -- make that first call outside a stream capture.
 * Nothing in it needs clearing between calls (every partial that is read was written by
 * the same call), but all calls on one GPU share it: calls that overlap in time on
 * different streams of one GPU race.
 */
int okv_sparse_attn_noalloc(const void* q, const void* k_base, const void* v_base,
                            const okv_kv_layout_t* layout, const int32_t* idx,
                            int64_t idx_stride, const int32_t* sel_lens, int32_t max_sel_len,
                            const void* tail_k, const void* tail_v, int64_t tail_token_stride,
                            int64_t tail_head_stride, int64_t tail_batch_stride,
                            const int32_t* tail_lens, int32_t max_tail_len, int32_t batch,
                            float scale, void* out, okv_stream_t stream);
int64_t okv_noalloc_scratch_bytes(void);

/*
 * Materialised gather: dst[b][j][g][:] = src[b][idx[b][j]][g][:] for j < sel_len_b,
 * dst addressed by (dst_token_stride, dst_head_stride, dst_batch_stride).
 * Replaces torch.index_select(cache, 2, idx) in set_idx_on_gpu
 * (modeling/spec_cache.py:298-303) for callers that need the gathered tensor
 * itself (a third-party attention consuming update()'s return value).
 */
int okv_gather_rows(const void* src_base, const okv_kv_layout_t* layout,
                    const int32_t* idx, int64_t idx_stride, const int32_t* sel_lens,
                    int32_t max_sel_len, int32_t batch, void* dst,
                    int64_t dst_token_stride, int64_t dst_head_stride,
                    int64_t dst_batch_stride, okv_stream_t stream);

/*
 * real_offload tier.  Copies the selected rows of one layer's K and V from PINNED
 * host memory (token-major rows of row_bytes bytes, row t at host_src + t*row_bytes)
 * into a contiguous device buffer, asynchronously on copy_stream, and records
 * done_event (a hipEvent_t, may be NULL) behind the copy.  host_idx is a HOST
 * array of n_rows ascending token indices.  Rows are packed by host_threads
 * CPU threads (>= 1; the call returns when packing is done) into host_staging
 * (pinned, >= n_rows*row_bytes) and moved with one hipMemcpyAsync.  The caller
 * must not reuse host_staging before done_event has completed.
 * Replaces `index_select(cpu cache, 2, idx.cpu()).cuda(non_blocking=True)`:
 * modeling/spec_cache.py:293-303.
 */
int okv_offload_stage(const void* host_src, int64_t row_bytes, const int32_t* host_idx,
                      int32_t n_rows, void* host_staging, int32_t host_threads,
                      void* dev_dst, okv_stream_t copy_stream, void* done_event);

/*
 * The per-token operations around the attention of a decode step, one launch each.  In the
 * reference these are third-party module calls (transformers 4.41.2 LlamaRMSNorm,
 * apply_rotary_pos_emb, LlamaMLP's act_fn(gate) * up) made from the layer forward,
 * modeling/omnikv.py:155-156 (input_layernorm), :219-227 (self_attn: projections + rotary
 * embedding), :228-236 (residual add, post_attention_layernorm, mlp); each is a chain of five
 * to ten elementwise launches there.  All tensors contiguous, same `dtype` (okv_dtype); every
 * intermediate is rounded to that type where the op-by-op chain rounds it.
 *   okv_rmsnorm   h = x, or x + residual rounded to dtype and written to sum_out (the new
 *                 residual stream) when residual != NULL;
 *                 out = weight * (h * rsqrt(mean(h^2) + eps)) with the normalised h rounded
 *                 to dtype before the product.  x, residual, sum_out, out: (rows, hidden).
 *   okv_rope      q_out[r][h] = q[r][h]*cos[r] + rotate_half(q[r][h])*sin[r], the same for k;
 *                 q row r at q + r*q_row_stride (num_q_heads*head_dim elements, the projection's
 *                 output), cos / sin (rows, head_dim), q_out (rows, num_q_heads, head_dim),
 *                 k_out (rows, num_kv_heads, head_dim); head_dim 128.
 *   okv_rope_append  okv_rope whose rotated k row, and the v row next to it, go straight into a
 *                 cache's K and V stores: row (request r, kv head h) to
 *                 store + r*store_batch_stride + h*store_head_stride + pos*store_token_stride
 *                 (strides in elements), pos = pos_dev[0] (device int64) when pos_dev != NULL.
 *                 Replaces the rotary embedding and the append of OmniKVMultiStageCache.update
 *                 for one new token (modeling/spec_cache.py:337-347,358-368).
 *   okv_silu_mul  out = silu(gate) * up over n elements.
 */
int okv_rmsnorm(const void* x, const void* residual, const void* weight, float eps, int32_t rows,
                int32_t hidden, int32_t dtype, void* sum_out, void* out, okv_stream_t stream);
int okv_rope(const void* q, int64_t q_row_stride, const void* k, int64_t k_row_stride,
             const void* cos, const void* sin, int32_t rows, int32_t num_q_heads,
             int32_t num_kv_heads, int32_t head_dim, int32_t dtype, void* q_out, void* k_out,
             okv_stream_t stream);
int okv_rope_append(const void* q, int64_t q_row_stride, const void* k, int64_t k_row_stride,
                    const void* v, int64_t v_row_stride, const void* cos, const void* sin,
                    int32_t rows, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                    int32_t dtype, void* q_out, void* k_store, void* v_store,
                    int64_t store_token_stride, int64_t store_head_stride,
                    int64_t store_batch_stride, const int64_t* pos_dev, int64_t pos,
                    okv_stream_t stream);
int okv_silu_mul(const void* gate, const void* up, int64_t n, int32_t dtype, void* out,
                 okv_stream_t stream);

/*
 * real_offload tier, incremental.  The rows staged on the device for a group of sparse
 * layers are a set -- attention over them does not depend on their order -- so a new selection
 * keeps the rows it shares with the previous one in place and fetches only the others, into
 * the slots the dropped rows free.  okv_offload_plan (once per selection; one workgroup, all
 * arrays in device memory) updates the two maps
 *   slot_tok[k]          token whose row sits in slot s, -1 for an empty slot
 *   slot_of[num_tokens]  slot of token t, -1 when it is not staged
 * (both filled with -1 before the first selection) from idx_new[k] (ascending, distinct,
 * < num_tokens) and writes the exchange: fetch_tok[r] -> slot fetch_slot[r] for
 * r < fetch_count[0], tokens ascending, slots ascending.  k <= 262144.  okv_offload_fetch
 * (once per layer of the group) then copies those rows: row fetch_tok[r] of src (rows of
 * row_bytes bytes, a multiple of 16; pinned host memory that the device can read, or device
 * memory) into row fetch_slot[r] of dev_dst.  max_rows (<= k) bounds the launch; the count
 * itself is read on the device, so both calls can be captured in a HIP graph.  The staged
 * buffer is then attended with okv_sparse_attn(idx = NULL, sel_len = k).
 * Replaces the full re-copy `index_select(cpu cache, 2, idx.cpu()).cuda()` that
 * set_idx_on_gpu repeats at every selection (modeling/spec_cache.py:293-303) and goes further
 * than the lazy variant, which can only skip a selection as a whole
 * (OmniKVLazyCache.set_out_idx, modeling/spec_cache.py:539-557).
 */
int okv_offload_plan(const int32_t* idx_new, int32_t k, int32_t* slot_tok, int32_t* slot_of,
                     int32_t num_tokens, int32_t* fetch_tok, int32_t* fetch_slot,
                     int32_t* fetch_count, okv_stream_t stream);
int okv_offload_fetch(const void* src, int64_t row_bytes, const int32_t* fetch_tok,
                      const int32_t* fetch_slot, const int32_t* fetch_count, int32_t max_rows,
                      void* dev_dst, okv_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* OMNIKV_HIP_H */
