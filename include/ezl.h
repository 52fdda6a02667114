/* C ABI of libezl: gfx950 kernels for the llama decoder-layer training step at TP=1.
 *
 * The reference (ModelTC/EasyLLM) has no FFI of its own for this path: its GPU kernels are reached
 * through optional Python imports (flash-attn, dropout_layer_norm, torch.matmul).  Each entry point
 * below names the reference call it stands in for (paths relative to the reference tree).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; buffers are owned by the caller;
 *     nothing here allocates or frees device memory; workspaces are passed in (one exception:
 *     ezl_rmsnorm_bwd_noalloc keeps its workspace in a device array of the library itself);
 *   - bf16 tensors: base 16-byte aligned, innermost dimension contiguous and a multiple of 8;
 *   - `stream` is a hipStream_t (NULL = default stream); all work is enqueued there, no host sync;
 *   - return 0 on success, a negative EZL_E* code otherwise; ezl_last_error() returns the message
 *     of the last failure on the calling thread;
 *   - re-entrant: no global mutable state; callable from any host thread (autograd workers included).
 *     The exception again is ezl_rmsnorm_bwd_noalloc, whose calls on one GPU share one array.
 *   - the code object is gfx950 only (64-wide waves, 160 KiB of LDS per workgroup; several kernels use
 *     more than 64 KiB): on any other GPU the first launch fails with EZL_EHIP.
 */
#ifndef EZL_H
#define EZL_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define EZL_OK 0
#define EZL_EINVAL (-1)       /* bad pointer / size / alignment */
#define EZL_EUNSUPPORTED (-2) /* shape or dtype outside what the kernels cover */
#define EZL_EHIP (-3)         /* the HIP runtime refused the launch */

int ezl_version(void);
const char* ezl_last_error(void);

/* ---- RMSNorm: base_modules/layers/fused_layer_norm.py:49-71 (flash_attn rms_norm seam :56-57) ----
 * y = (x [+ residual]) * rsqrt(mean(.^2) + eps) * weight, rows of h bf16 (h % 8 == 0, h <= 32768; rows wider than 8192,
 * which the reference hands to its unfused path (:56, :68-71), are read twice).
 * residual/sum_out are both NULL or both given (the residual add of llama/transformer.py:786 fused
 * in; sum_out receives x + residual rounded to bf16).  rstd: fp32 [rows], kept for backward. */
int ezl_rmsnorm_fwd(const void* x, const void* residual, const void* weight, void* y, void* sum_out, void* rstd,
                    int64_t rows, int64_t h, float eps, void* stream);
int64_t ezl_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t h);
/* dx = d/dx of the above (+ dresidual if given); dw goes to exactly one of dw_bf16 [h] (overwritten)
 * or dw_f32 [h] (overwritten, or added to when accumulate != 0). */
int ezl_rmsnorm_bwd(const void* dy, const void* x, const void* weight, const void* rstd, const void* dresidual, void* dx,
                    void* dw_bf16, void* dw_f32, int accumulate, void* workspace, int64_t workspace_bytes, int64_t rows,
                    int64_t h, void* stream);

/* ezl_rmsnorm_bwd without the workspace argument.  No counterpart in the reference: it exists for callers that cannot
 * obtain device memory at the call site (code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation).  The per-block dw partials go to a device array built into the library (16 MiB per GPU, held until the
 * process ends), which covers rows up to h = ezl_rmsnorm_bwd_noalloc_max_h() = 8192 (every layer width of the presets); a
 * larger h is refused with EZL_EUNSUPPORTED.  Same kernels and bit-identical results as ezl_rmsnorm_bwd.  All calls on one GPU
 * share the array: calls that overlap on one GPU (other streams or host threads) race.  The first call on a device looks
 * the array's address up (hipGetSymbolAddress) and is refused with EZL_EINVAL while `stream` is recording a graph. */
int64_t ezl_rmsnorm_bwd_noalloc_max_h(void);
int ezl_rmsnorm_bwd_noalloc(const void* dy, const void* x, const void* weight, const void* rstd, const void* dresidual, void* dx,
                            void* dw_bf16, void* dw_f32, int accumulate, int64_t rows, int64_t h, void* stream);

/* ---- SwiGLU: llama/transformer.py:220-222 + base_modules/layers/glu_activations.py:56-61 ---- */
int ezl_swiglu_fwd(const void* gate, const void* up, void* out, int64_t n, void* stream);
int ezl_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup, int64_t n, void* stream);

/* ---- rotary embedding: llama/positional_embeddings.py:17-36 (table), :94-96,105-122 (apply) ----
 * table: cos/sin fp32 [npos, half_dim], theta = (p / scale_factor) * inv_freq[j].
 * apply: x/out bf16 [s*b rows (s-major), nheads, d] with row strides in elements (out may alias x);
 * position_ids int64 [b, s] or NULL (position = s index); backward != 0 rotates by -theta. */
int ezl_rope_table(const void* inv_freq, void* cos_out, void* sin_out, int64_t npos, int64_t half_dim, float scale_factor,
                   void* stream);
int ezl_rope_apply(const void* x, void* out, const void* cos_table, const void* sin_table, const void* position_ids, int64_t s,
                   int64_t b, int64_t nheads, int64_t d, int64_t in_row_stride, int64_t out_row_stride, int64_t npos,
                   int backward, void* stream);
/* range test of the position ids that index the tables (the reference's cos[position_ids], positional_embeddings.py:109-117,
 * fails on an index past the table): ORs 1 into *bad_flag (device int32) if some id >= limit, 2 if some id < 0.  The apply
 * kernels themselves clamp. */
int ezl_ids_in_range(const void* ids_i64, int64_t n, int64_t limit, void* bad_flag, void* stream);
/* the same rotation of q [.., nq, d] and k [.., nk, d] of one layer (llama/transformer.py:437-448) in one launch */
int ezl_rope_apply_pair(const void* q, void* q_out, int64_t nq, int64_t q_in_stride, int64_t q_out_stride, const void* k,
                        void* k_out, int64_t nk, int64_t k_in_stride, int64_t k_out_stride, const void* cos_table,
                        const void* sin_table, const void* position_ids, int64_t s, int64_t b, int64_t d, int64_t npos,
                        int backward, void* stream);

/* ---- token embedding: base_modules/layers/vocab_parallel_emb.py:106-137 (F.embedding, TP=1) ----
 * gather: out[r] = weight[ids[r]] (bit-exact row copy); an id outside [0, vocab) ORs 1 (id >= vocab)
 * or 2 (id < 0) into *bad_flag (device int32) and yields a zero row.
 * scatter_add: dweight_f32[id] (+)= sum of dy[r] over rows with ids[r] == id, fp32, added in increasing row order whatever
 * the launch does (bit-reproducible).  accumulate != 0 adds to what the buffer holds; accumulate == 0 overwrites it and
 * zero-fills the rows of ids that do not occur, so the whole [vocab, h] gradient is written by the call.  Work is linear
 * in `rows`; an id that occurs n > 1024 times is summed by one workgroup in n consecutive row visits.  workspace:
 * ezl_embed_scatter_add_workspace_bytes(rows, vocab) bytes of device memory, 4-byte aligned, contents irrelevant before
 * and after. */
int ezl_embed_gather(const void* ids, const void* weight, void* out, void* bad_flag, int64_t rows, int64_t h, int64_t vocab,
                     void* stream);
int64_t ezl_embed_scatter_add_workspace_bytes(int64_t rows, int64_t vocab);
int ezl_embed_scatter_add(const void* ids, const void* dy, void* dweight_f32, void* workspace, int64_t workspace_bytes,
                          int64_t rows, int64_t h, int64_t vocab, int accumulate, void* stream);

/* ---- layout / dtype plumbing of llama/llama.py:145-188 (transpose, undo, float16_to_fp32) ---- */
int ezl_transpose01(const void* x, void* y, int64_t d0, int64_t d1, int64_t inner, void* stream); /* y[j,i,:] = x[i,j,:] */
int ezl_add(const void* a, const void* b, void* out, int64_t n, void* stream); /* residual add, transformer.py:797 */
int ezl_cast_bf16_to_f32(const void* in, void* out, int64_t n, void* stream);
int ezl_cast_f32_to_bf16(const void* in, void* out, int64_t n, void* stream);

/* ---- linear layers: column_parallel_linear.py:42 (fwd), :68 (dgrad), :99 (wgrad);
 *      row_parallel_linear.py:113; llama/lm_head.py:62 ----
 * C[M,N] (=|+=) A * B, bf16 operands, fp32 accumulation.
 *   A: a_kc ? A[m*lda + k] : A[k*lda + m]     B: b_kc ? B[n*ldb + k] : B[k*ldb + n]
 * out_dtype 0 = bf16, 1 = fp32.
 * workspace (optional, may be NULL): ezl_gemm_workspace_bytes(M, N, K) bytes of device memory, 16-byte aligned.  With it, a
 * tile count that leaves the last round of workgroups mostly empty (320 output tiles of 256 x 256 on 256 CUs, or 64 tiles
 * in all) is evened out: the reduction of those last tiles is split over several workgroups whose fp32 partial tiles are
 * added in a fixed order.  Without it the same result is computed by one workgroup per tile. */
int64_t ezl_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int ezl_gemm_bf16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                  int a_kc, int b_kc, int out_dtype, int accumulate, void* workspace, int64_t workspace_bytes, void* stream);
/* C (=|+=) sum_i A[i] * B[i] over `count` operand pairs with common M, N and leading dimensions and reduction lengths K[i]:
 * the input gradient sum_i dy_i W_i of the linears that share one input -- q/k/v (transformer.py:419-426) and gate/up
 * (:217-221), which the reference leaves to autograd as one matmul per linear (column_parallel_linear.py:68) plus adds.
 * One launch (fp32 sum, one rounding) for up to three pairs in the dgrad form; otherwise accumulating ezl_gemm_bf16 calls.
 * workspace as for ezl_gemm_bf16, sized by ezl_gemm_workspace_bytes(M, N, sum of K[i]). */
int ezl_gemm_bf16_ksplit(int count, const void* const* A, const void* const* B, void* C, int64_t M, int64_t N, const int64_t* K,
                         int64_t lda, int64_t ldb, int64_t ldc, int a_kc, int b_kc, int out_dtype, int accumulate, void* workspace,
                         int64_t workspace_bytes, void* stream);

/* bias of a linear layer: column_parallel_linear.py:43-44 (out = x + bias) and :100 (db = sum_rows dy);
 * db goes to exactly one of db_bf16 [n] or db_f32 [n] (added to when accumulate != 0). */
int ezl_bias_add(const void* x, const void* bias, void* out, int64_t rows, int64_t n, void* stream);
int64_t ezl_bias_grad_workspace_bytes(int64_t rows, int64_t n);
int ezl_bias_grad(const void* dy, void* db_bf16, void* db_f32, int accumulate, void* workspace, int64_t workspace_bytes,
                  int64_t rows, int64_t n, void* stream);

/* ---- attention: FlashAttention.forward, llama/transformer.py:83-143 (flash_attn_varlen_* seams
 *      :106-115) ----
 * q [T, nq, d], k/v [T, nk, d] bf16, d in {64, 128}; token n lives at
 * (n / s_len) * batch_stride + (n % s_len) * seq_stride (elements) + head * d.
 * cu_seqlens: int32 [ndocs + 1] or NULL (documents = the T / s_len batch rows; pass ndocs = T / s_len).
 * lse / delta: fp32 [nq, T] (delta = rowsum(dout * out) is produced by the backward call: scratch of the caller's).
 * strides (HOST pointer): fwd 8 values  q,k,v,out x (seq, batch); bwd 16 values: the same 8, then dout, dq, dk, dv x
 * (seq, batch).  Backward workspace: ezl_attn_bwd_workspace_bytes() bytes, 16-byte aligned (0 for MHA: may be NULL); with
 * a GQA group the query heads of a kv head are dealt to several workgroups whose fp32 partial dK / dV it holds, added in a
 * fixed order (results are bit-reproducible). */
int ezl_attn_fwd(const void* q, const void* k, const void* v, void* out, void* lse, const void* cu_seqlens, int64_t ndocs,
                 int64_t total_tokens, int64_t s_len, int64_t nq, int64_t nk, int64_t d, float scale, const int64_t* strides,
                 void* stream);
int64_t ezl_attn_bwd_workspace_bytes(int64_t total_tokens, int64_t ndocs, int64_t nq, int64_t nk, int64_t d);
int ezl_attn_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout, const void* lse, void* delta,
                 void* dq, void* dk, void* dv, const void* cu_seqlens, int64_t ndocs, int64_t total_tokens, int64_t s_len,
                 int64_t nq, int64_t nk, int64_t d, float scale, const int64_t* strides, void* workspace,
                 int64_t workspace_bytes, void* stream);

/* ---- unpadding by a key-padding mask: FlashAttention.forward, llama/transformer.py:117-141 (unpad_input / pad_input) ----
 * mask_compact: mask uint8 / bool [rows, s_len], non-zero = keep.  idx int32 [rows * s_len]: flat index of the p-th kept
 *   token (-1 past the last one); inv int32 [rows * s_len]: position of each token among the kept ones or -1;
 *   cu_seqlens int32 [rows + 1]: kept tokens before each row's end (the documents of the unpadded batch).
 * rows_gather: out row r = src row idx[r], zeros where idx[r] < 0 or >= n_src; rows of `width` bf16; row number n lives at
 *   (n / s_len) * batch_stride + (n % s_len) * seq_stride elements on either side.  With idx it unpads, with inv it pads
 *   back (masked positions become zero rows); each is the other's backward. */
int ezl_mask_compact(const void* mask_u8, int64_t rows, int64_t s_len, void* idx, void* inv, void* cu_seqlens, void* stream);
int ezl_rows_gather(const void* src, const void* idx, void* out, int64_t n_out, int64_t width, int64_t n_src, int64_t src_s_len,
                    int64_t src_seq_stride, int64_t src_batch_stride, int64_t out_s_len, int64_t out_seq_stride,
                    int64_t out_batch_stride, void* stream);

/* ---- loss: base_modules/functions/cross_entropy.py:24-112 and llama/losses.py:20-56 ----
 * logits [rows, vocab] bf16 (dtype 0) or fp32 (dtype 1); labels int64 [rows]; a label outside
 * [0, vocab - cut_size) is masked exactly as the reference does (pred = 0, no one-hot).
 * prepare: weights[i] = loss_mask[i] * (labels[i] != ignore_index), count[0] = sum(weights);
 *          mask_dtype 0 none(=1), 1 fp32, 2 bool/uint8, 3 int64, 4 bf16.
 * fwd/bwd: the reference's per-token autograd function split in two (loss + logsumexp; grad).
 * fused:   loss rows and grad = (softmax - onehot) * weights / count in ONE visit (grad may alias logits).
 * reduce:  loss_out[0] = sum(loss_rows * weights) / count[0]. */
int ezl_ce_prepare(const void* labels, const void* loss_mask, int mask_dtype, int64_t ignore_index, void* weights, void* count,
                   int64_t n, void* stream);
int ezl_ce_fwd(const void* logits, const void* labels, void* loss, void* lse, int64_t rows, int64_t vocab, int64_t cut_size,
               int dtype, void* stream);
int ezl_ce_bwd(const void* logits, const void* labels, const void* lse, const void* grad_out, void* grad, int64_t rows,
               int64_t vocab, int64_t cut_size, int dtype, void* stream);
int ezl_ce_fused(const void* logits, const void* labels, const void* weights, const void* count, void* loss_rows, void* grad,
                 int64_t rows, int64_t vocab, int64_t cut_size, int dtype, void* stream);
int ezl_ce_reduce(const void* loss_rows, const void* weights, const void* count, void* loss_out, int64_t n, void* stream);
/* x *= scalar[0] unless scalar[0] == 1 (applies the upstream gradient of the fused loss) */
int ezl_scale_by_scalar(void* x, const void* scalar_f32, int64_t n, int dtype, void* stream);

/* ---- optimizer step: apex FusedAdam in AdamW mode under DeepSpeed's bf16 optimizer with gradient clipping
 *      (llm/utils/model/optimizer_helper.py:70-98; configs/megatron/llama_7b_sft.yaml:13,106-112) ----
 * sumsq:     partials[0 .. ezl_sumsq_partials()) = per-block sums of x[i]^2 (fp32 x, every slot written).
 * clip_coef: norm_coef_out[0] = sqrt(sum of `count` partials) (fixed order), norm_coef_out[1] = max_norm / (norm + 1e-6)
 *            if that is < 1, else 1 (max_norm <= 0: no clipping).
 * adamw:     g = grad * norm_coef[1] (1 if norm_coef is NULL); m = b1 m + (1-b1) g; v = b2 v + (1-b2) g^2;
 *            master -= lr * (m/bc1 / (sqrt(v/bc2) + eps) + weight_decay * master), bc = 1 - beta^step (1 without bias
 *            correction); param_bf16 (may be NULL) = round-to-nearest-even of the new master value. */
int64_t ezl_sumsq_partials(void);
int ezl_sumsq_f32(const void* x, int64_t n, void* partials, void* stream);
int ezl_clip_coef(const void* partials, int64_t count, float max_norm, void* norm_coef_out, void* stream);
int ezl_adamw_step(void* master, void* exp_avg, void* exp_avg_sq, const void* grad, void* param_bf16, int64_t n, float lr,
                   float beta1, float beta2, float eps, float weight_decay, int64_t step, int bias_correction,
                   const void* norm_coef, void* stream);

/* ---- packed-sequence sample index (host code, no GPU): llm/data/cores/helpers.cpp:36-122 `build_location_idx`
 *      (python twin llm/data/nlp_dataset.py:424-463) ----
 * rows:  (num_epochs * tokens_per_epoch - 1) / seq_length + 1, or -1 for arguments the reference asserts against.
 * build: out[k] = (position in doc_idx, token offset in that document) of the first token of sample k, samples being
 *        seq_length + 1 tokens long and overlapping by one token; int32 [rows][2].  All indices are bounds-checked. */
int64_t ezl_location_idx_rows(int64_t seq_length, int64_t num_epochs, int64_t tokens_per_epoch);
int ezl_build_location_idx(const int32_t* sizes, int64_t n_sizes, const int32_t* doc_idx, int64_t n_doc_idx, int64_t seq_length,
                           int64_t num_epochs, int64_t tokens_per_epoch, int32_t* out, int64_t out_rows);

#ifdef __cplusplus
}
#endif
#endif
