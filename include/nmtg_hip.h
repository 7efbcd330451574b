/*
 * nmtg_hip.h — C ABI of libnmtg_hip.so: MI355X (gfx950) kernels for the fused transformer-layer
 * ops of NMTGMinor (LayerNorm, fused MLP, self / encoder-decoder attention, masked softmax +
 * dropout, dropout + residual add, label-smoothed softmax cross-entropy).
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers owned by the caller. The library never allocates, frees
 *     or keeps device memory, and holds no state between calls apart from the last error text.
 *   - Tensors are dense row-major unless a leading dimension / stride argument says otherwise.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream). Calls only enqueue
 *     work on that stream; they never synchronise the device.
 *   - Element types are named by nmtg_dtype codes.
 *   - Return value: 0 on success, a negative nmtg_status otherwise; nmtg_last_error() then
 *     returns a human-readable reason (thread-local). No entry point aborts or exits.
 *
 * Each declaration cites the interface of the reference tree (paths relative to the NMTGMinor
 * checkout) that it stands in for.
 */
#ifndef NMTG_HIP_H_
#define NMTG_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { NMTG_F32 = 0, NMTG_F16 = 1, NMTG_BF16 = 2 } nmtg_dtype;

typedef enum {
  NMTG_OK = 0,
  NMTG_ERR_INVALID = -1,     /* bad argument: shape, dtype, alignment, null pointer */
  NMTG_ERR_UNSUPPORTED = -2, /* valid request that this build has no kernel for */
  NMTG_ERR_LAUNCH = -3       /* HIP reported an error when the kernel was enqueued */
} nmtg_status;

/* Activation codes of the fused MLP. Reference: the per-activation extension modules
 * onmt/modules/extensions/mlp/mlp_{relu,gelu,silu,agelu}.cpp and the plain mlp.cpp. */
typedef enum {
  NMTG_ACT_NONE = 0,
  NMTG_ACT_RELU = 1,
  NMTG_ACT_GELU = 2,  /* exact erf form */
  NMTG_ACT_SILU = 3,
  NMTG_ACT_AGELU = 4  /* tanh approximation, 0.044715 */
} nmtg_act;

/* Library version (major*10000 + minor*100 + patch) and the last error of the calling thread. */
int nmtg_version(void);
const char* nmtg_last_error(void);

/* ------------------------------------------------------------------------------------------
 * LayerNorm.
 * Reference: fast_layer_norm_cuda.ln_fwd / ln_bwd,
 *   onmt/modules/extensions/layer_norm/ln_api.cpp:80-153 (ln_fwd), :156-249 (ln_bwd).
 *
 * x [rows, hidden] of in_dtype; gamma, beta [hidden] of w_dtype; z [rows, hidden] of w_dtype
 * (the reference forms the output in the weight dtype); mu, rsigma [rows] fp32.
 * Any hidden size is accepted (the reference registers 25 sizes, ln_fwd_cuda_kernel.cu:73-233).
 * ------------------------------------------------------------------------------------------ */
int nmtg_ln_fwd(const void* x, const void* gamma, const void* beta, void* z, float* mu,
                float* rsigma, int64_t rows, int64_t hidden, float eps, int in_dtype, int w_dtype,
                void* stream);

/* Number of partial rows ln_bwd writes: dgamma_part / dbeta_part are [n_part, hidden] fp32
 * (the reference's ctas_per_col, ln_api.cpp:214-215). */
int64_t nmtg_ln_bwd_parts(int64_t rows, int64_t hidden);

/* dz [rows, hidden] w_dtype; x_or_z [rows, hidden] in_dtype (x, or z when memory_efficient);
 * mu may be NULL and beta is required when memory_efficient != 0; dx [rows, hidden] in_dtype;
 * dgamma, dbeta [hidden] w_dtype; dgamma_part, dbeta_part [n_part, hidden] fp32 workspace that
 * is also an output, with n_part == nmtg_ln_bwd_parts(rows, hidden). */
int nmtg_ln_bwd(const void* dz, const void* x_or_z, const float* mu, const float* rsigma,
                const void* gamma, const void* beta, void* dx, void* dgamma, void* dbeta,
                float* dgamma_part, float* dbeta_part, int64_t n_part, int64_t rows,
                int64_t hidden, int memory_efficient, int in_dtype, int w_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dropout + residual add (in place) and its backward.
 * Reference: fused_dropout_add_cuda.forward(is_training, x, residual, p) -> (mask, out) and
 *   .backward(grad, mask, p) -> dx,
 *   onmt/modules/extensions/dropout_add/fused_dropout_add_cuda_kernel.cu:19-66 and :68-95.
 *
 * x <- residual + x * keep / (1 - p), n elements, in place in x (as the reference does).
 * mask_mode: 0 = no dropout (x <- x + residual, mask untouched; the reference's eval / p == 0
 *            branch), 1 = read the keep mask from `mask` (replay), 2 = draw the keep mask from
 *            Philox4x32-10 keyed by (seed, offset, element index) and write it to `mask`.
 * mask: n bytes, 1 = keep.
 * ------------------------------------------------------------------------------------------ */
int nmtg_dropout_add_fwd(void* x, const void* residual, uint8_t* mask, int64_t n, float p,
                         int mask_mode, uint64_t seed, uint64_t offset, int dtype, void* stream);

/* grad_x <- grad_out * mask / (1 - p); the residual's gradient is grad_out itself. */
int nmtg_dropout_add_bwd(const void* grad_out, const uint8_t* mask, void* grad_x, int64_t n,
                         float p, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Masked softmax over the last dimension with optional inverted dropout.
 * Reference: the softmax stage of the fused attention, dispatch_softmax_dropout /
 *   dispatch_softmax / dispatch_softmax_dropout_presampled
 *   (onmt/modules/extensions/multihead_attn_blaslt/softmax_apex.h:443-486, :1263-1300, :874-912),
 *   backward dispatch_softmax_dropout_backward_recompute / dispatch_softmax_backward_norecompute
 *   (:4039-4075, :3467-3500); stand-alone callers use the module mask_softmax_dropout_cuda
 *   (onmt/modules/optimized/attention_softmax.py:32-59).
 *
 * scores [rows, cols]; rows = batch * heads * q_len. key_mask (1 = masked key, may be NULL):
 *   mask_kind 0 none, 1 key padding [batch, cols], 2 time mask [q_len, cols]. Scores may also
 *   already hold -inf. A row with every key masked gives zeros.
 * softmax_out (may be NULL) receives the probabilities before dropout, dropped_out the result.
 * dropout_mode 0 none, 1 replay `dropout_mask` [rows, cols], 2 draw it from Philox and store it.
 * Rows of up to 4096 keys (16-bit, cols % 8 == 0) / 2048 keys otherwise; the reference's limit is
 *   2048 (softmax_apex.h:450-452).
 * ------------------------------------------------------------------------------------------ */
int nmtg_softmax_dropout_fwd(const void* scores, const uint8_t* key_mask, int mask_kind,
                             void* softmax_out, void* dropped_out, uint8_t* dropout_mask,
                             int dropout_mode, float p, uint64_t seed, uint64_t offset,
                             int64_t rows, int64_t cols, int64_t q_len, int64_t heads, int dtype,
                             void* stream);

/* grad_scores = P * (g - sum_k P * g), g = dropout_mask * grad_dropped / (1 - p).
 * saved holds the (masked) scores when saved_is_scores != 0 — P is recomputed, the reference's
 * "backward_recompute" — or the probabilities P themselves. dropout_mode 0 or 1. */
int nmtg_softmax_dropout_bwd(const void* grad_dropped, const void* saved, int saved_is_scores,
                             const uint8_t* key_mask, int mask_kind, const uint8_t* dropout_mask,
                             int dropout_mode, float p, void* grad_scores, int64_t rows,
                             int64_t cols, int64_t q_len, int64_t heads, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Label-smoothed softmax cross-entropy.
 * Reference: xentropy_cuda.forward(logits, labels, smoothing, half_to_float) ->
 *   (losses, max_log_sum_exp) and .backward(grad_loss, logits, max_log_sum_exp, labels,
 *   smoothing) -> grad_logits, onmt/modules/extensions/xentropy/interface.cpp:24-47,
 *   xentropy_kernel.cu:571-718; the padding masked_fill_ of the Python wrapper
 *   (onmt/modules/optimized/softmax_xentropy.py:10,24) is folded in through padding_idx
 *   (pass a value no label takes, e.g. INT64_MIN, to switch it off).
 *
 * logits [rows, vocab] (fp32 / fp16 / bf16) with row pitch ld_logits >= vocab elements (the
 * reference's tensors are dense: ld_logits = vocab), labels int64 [rows]; losses, lse fp32 [rows];
 * grad_loss fp32 [rows]; grad_logits [rows, vocab] in the logits dtype with row pitch ld_grad;
 * elements between vocab and the pitch are neither read nor written. fp32 accumulation.
 * The backward is elementwise once lse is known, so it also works on a slice of the classes:
 * the `vocab` columns handed in are classes [class_offset, class_offset + vocab) of
 * total_classes (labels stay global; smoothing spreads over total_classes). The whole row:
 * class_offset = 0, total_classes = vocab. grad_logits may be the logits buffer itself (same
 * pitch): every element is read before it is overwritten. (The reference allocates a second
 * tensor of the logits' size, xentropy_kernel.cu:636-645.)
 * ------------------------------------------------------------------------------------------ */
int nmtg_xentropy_fwd(const void* logits, const int64_t* labels, float* losses, float* lse,
                      int64_t rows, int64_t vocab, int64_t ld_logits, float smoothing,
                      int64_t padding_idx, int dtype, void* stream);

/* nmtg_xentropy_fwd that also writes argmax [rows] (int64): the index of each row's largest logit with
 * torch.argmax's rule (NaN counts as the largest value; the lowest index among equals). Replaces the
 * argmax over the logits in the reference's evaluation branch (NMTLossFunc.forward,
 * onmt/modules/loss.py:293-311), which re-reads the whole logits tensor. */
int nmtg_xentropy_fwd_argmax(const void* logits, const int64_t* labels, float* losses, float* lse,
                             int64_t* argmax, int64_t rows, int64_t vocab, int64_t ld_logits,
                             float smoothing, int64_t padding_idx, int dtype, void* stream);

int nmtg_xentropy_bwd(const float* grad_loss, const void* logits, const float* lse,
                      const int64_t* labels, void* grad_logits, int64_t rows, int64_t vocab,
                      int64_t ld_logits, int64_t ld_grad, int64_t class_offset,
                      int64_t total_classes, float smoothing, int64_t padding_idx, int dtype,
                      void* stream);

/* ------------------------------------------------------------------------------------------
 * Strided-batched GEMM on the MFMA units (fp16 / bf16 in and out, fp32 accumulation), row-major:
 *   C[b] = alpha * op(A[b]) * op(B[b]) (+ bias[n]),   op(A) is m x k, op(B) is k x n.
 *   trans_a == 0: A stored [m, k] (lda >= k);  trans_a != 0: A stored [k, m] (lda >= m).
 *   trans_b == 0: B stored [k, n] (ldb >= n);  trans_b != 0: B stored [n, k] (ldb >= k).
 *   (trans_a, trans_b) = (0,1), (0,0), (1,0) are provided; these are the products the path uses.
 * Reference: the cuBLAS / cuBLASLt calls behind the fused ops — mlp_gemm
 *   (onmt/modules/extensions/mlp/mlp_gelu_cuda.cu:86-201), gemm_bias_lt
 *   (multihead_attn_blaslt/gemm_blaslt.cuh:9-54) and the strided-batched wrapper
 *   (multihead_attn_blaslt/strided_batched_gemm_blaslt.cuh:9-126); also linear_blaslt
 *   (mlp_blaslt/linear.cpp:142-144).
 * workspace (may be NULL): fp32 scratch of nmtg_gemm_workspace_bytes(m, n, k, batch) bytes; with
 *   it a (1,0) product with a long reduction is split over the chip (deterministic reduction).
 * ------------------------------------------------------------------------------------------ */
int64_t nmtg_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k, int64_t batch);

int nmtg_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a,
              int64_t lda, int64_t stride_a, const void* b, int64_t ldb, int64_t stride_b, void* c,
              int64_t ldc, int64_t stride_c, int64_t batch, const void* bias, void* workspace,
              int64_t workspace_bytes, int dtype, void* stream);

/* nmtg_gemm without a workspace argument, for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. The split-K
 * partial sums go to an array of nmtg_gemm_static_max_workspace_bytes() (32 MiB) that the library keeps in device
 * memory on every GPU it runs on until the process ends; a shape whose nmtg_gemm_workspace_bytes() exceeds that is
 * rejected with NMTG_ERR_INVALID. The call itself allocates and frees nothing. All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams) race. Results are bit-identical to nmtg_gemm with a
 * workspace. */
int64_t nmtg_gemm_static_max_workspace_bytes(void);
int nmtg_gemm_static(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a,
                     int64_t lda, int64_t stride_a, const void* b, int64_t ldb, int64_t stride_b, void* c,
                     int64_t ldc, int64_t stride_c, int64_t batch, const void* bias, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Fused MLP: y = W_n(... dropout(act(W_1 x + b_1)) ...) + b_n, nn.Linear weight layout [out, in].
 * Reference: fused_mlp_gelu.forward / backward / backward_input_only
 *   (onmt/modules/extensions/mlp/mlp_gelu.cpp:69-127, :129-194, :197-264), the relu / silu / agelu
 *   siblings (mlp_relu.cpp:68-272, mlp_silu.cpp, mlp_agelu.cpp) and mlp_gelu_blaslt
 *   (mlp_blaslt/mlp_gelu.cpp:75-242).
 *
 * x [batch, in_features]; weights[i] [out_features[i], in_i]; biases (array or NULL; entries may be
 * NULL) [out_features[i]]; out [batch, out_features[n-1]].
 * post_acts / pre_acts: the hidden layers' dropped activations / pre-activations, concatenated
 *   layer after layer ([batch, out_features[0]], [batch, out_features[1]], ...) — the reference's
 *   reserved_space / reserved_activations. pre_acts may be NULL (relu keeps only the output).
 * mask: one byte per hidden activation in the same concatenated order, 1 = keep.
 *   mask_mode 0 no dropout, 1 replay `mask`, 2 draw it from Philox (seed, offset) and store it.
 * act: an nmtg_act code. dtype: NMTG_F16 or NMTG_BF16.
 * ------------------------------------------------------------------------------------------ */
int nmtg_mlp_fwd(int num_layers, const void* x, const void* const* weights,
                 const void* const* biases, const int64_t* out_features, int64_t batch,
                 int64_t in_features, void* out, void* post_acts, void* pre_acts, uint8_t* mask,
                 int mask_mode, float p, uint64_t seed, uint64_t offset, int act, int dtype,
                 void* stream);

int64_t nmtg_mlp_bwd_workspace_bytes(int num_layers, const int64_t* out_features, int64_t batch,
                                     int64_t in_features);
/* The same for a given element type: fp32 (the precision of the reference's own MLP tests,
 * onmt/modules/mlp/test_mlp_gelu.py:229-307) needs twice the room for the hidden gradients; the
 * function above sizes for the 16-bit types. */
int64_t nmtg_mlp_bwd_dtype_workspace_bytes(int num_layers, const int64_t* out_features,
                                           int64_t batch, int64_t in_features, int dtype);

/* grad_x may be NULL (the reference skips it when x does not require grad); grad_weights /
 * grad_biases may be NULL or hold NULL entries (backward_input_only). mask NULL or p == 0: no
 * dropout. With pre_acts == NULL and act == relu the gradient gate is taken from the dropped
 * output (mlp_relu_cuda.cu:1174-1240). workspace: nmtg_mlp_bwd_workspace_bytes(...) bytes,
 * 256-byte aligned. */
int nmtg_mlp_bwd(int num_layers, const void* x, const void* const* weights,
                 const int64_t* out_features, int64_t batch, int64_t in_features,
                 const void* grad_out, const void* post_acts, const void* pre_acts,
                 const uint8_t* mask, float p, int act, void* grad_x, void* const* grad_weights,
                 void* const* grad_biases, void* workspace, int64_t workspace_bytes, int dtype,
                 void* stream);

/* ------------------------------------------------------------------------------------------
 * Self-attention (time-first activations, per-head interleaved q/k/v).
 * Reference: self_multihead_attn_blaslt.forward / backward / forward_compact / backward_compact
 *   (onmt/modules/extensions/multihead_attn_blaslt/self_multihead_attn.cpp:95-132, :162-212,
 *   :135-160, :215-240; device side self_multihead_attn_cuda.cu:40-243, :413-742).
 *
 * x [T, B, E]; w_in [3E, E] with rows ordered (head, {q,k,v}, head_dim); w_out [E, E]; biases may
 * be NULL. lin [T, B, 3E] (= [T, B*H, 3, D]) is the input projection: written when x / w_in are
 * given, read when both are NULL (the "compact" form, projections done by the caller).
 * mask (1 = masked): mask_kind 0 none, 1 key padding [B, T], 2 time mask [T, T].
 * scores [B*H, T, T]: scaled, masked (-inf) pre-softmax scores; softmax_out (may be NULL) the
 * probabilities before dropout; dropped the probabilities after dropout (what multiplies v).
 * scores may be NULL for an inference call (dropout_mode 0, softmax_out NULL) with head dimension
 * 64 or 128 and a key count that is a multiple of 4: probabilities and context then come from one
 * kernel and no score tensor is written (the backward needs it, so a call that will be
 * back-propagated passes it); `dropped` may then be NULL too, for a caller that does not return
 * the probabilities (no [B*H, T, T] tensor at all). Same for nmtg_encdec_attn_fwd (its Tk then
 * has no upper limit).
 * dropout_mode 0 none, 1 replay dropout_mask [B*H, T, T], 2 draw it (Philox) and store it.
 * ctx [T, B, E]; out [T, B, E] (NULL together with w_out in the compact form).
 * dtype NMTG_F16 or NMTG_BF16 (the reference is fp16 only); T <= 4096.
 * ------------------------------------------------------------------------------------------ */
int nmtg_self_attn_fwd(const void* x, const void* w_in, const void* w_out, const void* b_in,
                       const void* b_out, const uint8_t* mask, int mask_kind, void* lin,
                       void* scores, void* softmax_out, void* dropped, uint8_t* dropout_mask,
                       int dropout_mode, float p, uint64_t seed, uint64_t offset, void* ctx,
                       void* out, int64_t t, int64_t b, int64_t e, int heads, int dtype,
                       void* stream);

int64_t nmtg_self_attn_bwd_workspace_bytes(int64_t t, int64_t b, int64_t e, int heads);

/* grad_out [T, B, E]: gradient of `out`, or of `ctx` in the compact form (w_out == NULL; then
 * ctx, x, w_in may be NULL and only grad_lin is produced). Any of grad_x, grad_w_*, grad_b_* may
 * be NULL to skip it. grad_lin (may be NULL): receives the gradient of `lin`, [T, B, 3E].
 * dropout_mask NULL or p == 0: no dropout was applied. The probabilities are recomputed from
 * `scores`. workspace: nmtg_self_attn_bwd_workspace_bytes bytes, 256-byte aligned. */
int nmtg_self_attn_bwd(const void* grad_out, const void* ctx, const void* dropped,
                       const void* scores, const void* lin, const void* x, const void* w_in,
                       const void* w_out, const uint8_t* dropout_mask, float p, void* grad_x,
                       void* grad_w_in, void* grad_w_out, void* grad_b_in, void* grad_b_out,
                       void* grad_lin, void* workspace, int64_t workspace_bytes, int64_t t,
                       int64_t b, int64_t e, int heads, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Encoder-decoder attention.
 * Reference: encdec_multihead_attn_bias_blaslt.forward / backward / forward_compact /
 *   backward_compact (multihead_attn_blaslt/encdec_multihead_attn_bias.cpp:124-173, :203-267,
 *   :175-201, :269-308; device side encdec_multihead_attn_bias_cuda.cu:40-273, :1089-1472).
 *
 * x_q [Tq, B, E], x_kv [Tk, B, E]; w_q [E, E]; w_kv [2E, E] with rows ordered (head, {k,v},
 * head_dim); q_lin [Tq, B, E], kv_lin [Tk, B, 2E] written (or read, when the matching input and
 * weight are NULL). pad_mask [B, Tk] (1 = masked) or NULL. Other arguments as for self-attention;
 * scores / dropped are [B*H, Tq, Tk]; Tk <= 4096.
 * ------------------------------------------------------------------------------------------ */
int nmtg_encdec_attn_fwd(const void* x_q, const void* x_kv, const void* w_q, const void* w_kv,
                         const void* w_out, const void* b_q, const void* b_kv, const void* b_out,
                         const uint8_t* pad_mask, void* q_lin, void* kv_lin, void* scores,
                         void* softmax_out, void* dropped, uint8_t* dropout_mask, int dropout_mode,
                         float p, uint64_t seed, uint64_t offset, void* ctx, void* out, int64_t tq,
                         int64_t tk, int64_t b, int64_t e, int heads, int dtype, void* stream);

int64_t nmtg_encdec_attn_bwd_workspace_bytes(int64_t tq, int64_t tk, int64_t b, int64_t e, int heads);

int nmtg_encdec_attn_bwd(const void* grad_out, const void* ctx, const void* dropped,
                         const void* scores, const void* q_lin, const void* kv_lin,
                         const void* x_q, const void* x_kv, const void* w_q, const void* w_kv,
                         const void* w_out, const uint8_t* dropout_mask, float p, void* grad_x_q,
                         void* grad_x_kv, void* grad_w_q, void* grad_w_kv, void* grad_w_out,
                         void* grad_b_q, void* grad_b_kv, void* grad_b_out, void* grad_q_lin,
                         void* grad_kv_lin, void* workspace, int64_t workspace_bytes, int64_t tq,
                         int64_t tk, int64_t b, int64_t e, int heads, int dtype, void* stream);

/* The backward of the bias-free extension, which saves the softmax results instead of the scores:
 * encdec_multihead_attn_cuda.backward(heads, output_grads, matmul2_results, dropout_results,
 * softmax_results, input_lin_q_results, input_lin_kv_results, inputs_q, inputs_kv, weights..., dropout_mask, p)
 * (call site onmt/modules/optimized/encdec_attention_func.py:322-345). As nmtg_encdec_attn_bwd with
 * `softmax_results` [B*H, Tq, Tk] (pre-dropout probabilities) in place of `scores`; nothing is
 * recomputed, there are no biases. Same workspace. */
int nmtg_encdec_attn_bwd_from_probs(const void* grad_out, const void* ctx, const void* dropped,
                                    const void* softmax_results, const void* q_lin,
                                    const void* kv_lin, const void* x_q, const void* x_kv,
                                    const void* w_q, const void* w_kv, const void* w_out,
                                    const uint8_t* dropout_mask, float p, void* grad_x_q,
                                    void* grad_x_kv, void* grad_w_q, void* grad_w_kv,
                                    void* grad_w_out, void* grad_q_lin, void* grad_kv_lin,
                                    void* workspace, int64_t workspace_bytes, int64_t tq,
                                    int64_t tk, int64_t b, int64_t e, int heads, int dtype,
                                    void* stream);

/* ------------------------------------------------------------------------------------------
 * Rotary position encoding of queries / keys, in place, and its transpose (backward).
 * Reference: apply_rotary_pos_emb / rotate_half / rotate_backward and their call sites
 *   (onmt/modules/optimized/self_attention_func.py:25-48, :178-184, :467-469;
 *   onmt/modules/optimized/encdec_attention_func.py:21-34), which run as PyTorch ops there.
 * x[pos * stride_t + head * stride_n + part * stride_part + j], j < d (d even), pos < t, head < n,
 * part < nparts (strides in elements): y = x cos + rotate_half(x) sin with cos, sin [t, d] in the
 * dtype of x; inverse != 0 applies the transpose, dx = g cos + rotate_backward(sin g). The query
 * and key slots of the head-interleaved projection [T, B*H, 3, D] are two parts of one call
 * (stride_t = B*H*3*D, stride_n = 3*D, stride_part = D).
 * ------------------------------------------------------------------------------------------ */
int nmtg_rotary(void* x, const void* cos_table, const void* sin_table, int64_t t, int64_t n,
                int64_t d, int64_t nparts, int64_t stride_t, int64_t stride_n, int64_t stride_part,
                int inverse, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Attention over packed variable-length sequences without a [heads, len_q, len_k] tensor.
 * Reference: flash_attn_cuda.fwd / .bwd as bound at onmt/modules/optimized/flash_mha.py:43-75
 *   (callers FlashAttnQKVPackedFunc / FlashAttnKVPackedFunc :104-183,
 *   onmt/models/speech_recognizer/whisper_encoder.py:329-356).
 * q [total_q, heads, head_dim], k / v [total_k, heads, head_dim], out like q: 16-bit views with a
 * contiguous head_dim (64 or 128), token and head strides in elements (multiples of 8), 16-byte
 * aligned (the slots of a packed [total, 3, heads, head_dim] projection qualify). Sequence b owns
 * tokens cu_seqlens[b] .. cu_seqlens[b+1]-1 (device int32 [batch + 1]); lengths must not exceed
 * max_seqlen_q / max_seqlen_k (longer ones are cut there). Per sequence and head:
 *   P = softmax_rows(softmax_scale * Q K^T)   (1e-6 <= |softmax_scale| <= 1e6; causal: keys j > i
 *   masked, aligned at the first token of both), out = (keep * P * dropout_scale) V, softmax_lse [batch, heads, max_seqlen_q]
 *   = log sum exp of the scaled scores (fp32; entries past a sequence's length are not written;
 *   -inf for a sequence without keys, whose out rows are 0).
 * dropout_mode 0: none. 1: replay dropout_mask (uint8 keep flags [batch, heads, max_seqlen_q,
 * max_seqlen_k]), scale 1 / (1 - p). 2: draw from Philox (seed, offset): element (i, j) is kept when
 * byte 4 (i % 4) + (j % 4) of block ((b heads + h) ceil(max_q / 4) + i / 4) ceil(max_k / 4) + j / 4
 * is below t = round(256 (1 - p)), scale 256 / t; dropout_mask_out, when not null, receives the
 * keep flags in the layout of dropout_mask. The backward regenerates the same mask from the same
 * (seed, offset).
 * dropout_bits (modes 1 and 2; may be NULL in mode 0): device workspace of
 * nmtg_flash_attn_dropout_bits_bytes(batch, heads, max_seqlen_q, max_seqlen_k) bytes, 16-byte
 * aligned. A small kernel ahead of the attention kernels fills it with the keep decisions, one bit
 * per element, and the attention kernels read only that (the generator's integer arithmetic would
 * otherwise cost them more than the softmax). A caller that keeps the workspace of the forward
 * call hands it to the backward with dropout_bits_ready = 1, which then neither runs the generator
 * nor reads dropout_mask; with 0 the backward fills it again from (seed, offset) or the mask.
 * nmtg_flash_attn_bwd: dq, dk, dv in views like q, k, v (every row of every sequence written),
 * softmax_d [batch, heads, max_seqlen_q] = rowsum(dout * out) (fp32, written). Deterministic: no
 * atomics.
 * ------------------------------------------------------------------------------------------ */
int64_t nmtg_flash_attn_dropout_bits_bytes(int64_t batch, int64_t heads, int64_t max_seqlen_q,
                                           int64_t max_seqlen_k);

int nmtg_flash_attn_fwd(const void* q, const void* k, const void* v, void* out,
                        const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, float* softmax_lse,
                        int64_t batch, int64_t heads, int64_t head_dim, int64_t max_seqlen_q,
                        int64_t max_seqlen_k, int64_t q_stride_t, int64_t q_stride_h,
                        int64_t k_stride_t, int64_t k_stride_h, int64_t v_stride_t, int64_t v_stride_h,
                        int64_t out_stride_t, int64_t out_stride_h, float softmax_scale, int causal,
                        int dropout_mode, float dropout_p, const uint8_t* dropout_mask,
                        uint8_t* dropout_mask_out, void* dropout_bits, uint64_t seed, uint64_t offset,
                        int dtype, void* stream);

int nmtg_flash_attn_bwd(const void* dout, const void* q, const void* k, const void* v,
                        const void* out, const float* softmax_lse, void* dq, void* dk, void* dv,
                        float* softmax_d, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                        int64_t batch, int64_t heads, int64_t head_dim, int64_t max_seqlen_q,
                        int64_t max_seqlen_k, int64_t dout_stride_t, int64_t dout_stride_h,
                        int64_t q_stride_t, int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_h,
                        int64_t v_stride_t, int64_t v_stride_h, int64_t out_stride_t,
                        int64_t out_stride_h, int64_t dq_stride_t, int64_t dq_stride_h,
                        int64_t dk_stride_t, int64_t dk_stride_h, int64_t dv_stride_t,
                        int64_t dv_stride_h, float softmax_scale, int causal, int dropout_mode,
                        float dropout_p, const uint8_t* dropout_mask, void* dropout_bits,
                        int dropout_bits_ready, uint64_t seed, uint64_t offset, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * The same kernels over a padded batch: the training call of the attention core when nobody reads
 * the probabilities.
 * Reference: the core of SelfAttnFunc / EncdecAttnFunc between the two projections
 *   (onmt/modules/optimized/self_attention_func.py:136-283 forward, :296-520 backward;
 *   encdec_attention_func_bias.py:20-213), whose [heads, len_q, len_k] score, probability and
 *   dropout tensors exist only for the backward and for return_coverage.
 * q [len_q, batch, heads, head_dim], k / v [len_k, batch, heads, head_dim], out like q: 16-bit views
 * with a contiguous head_dim (64 or 128) and position, batch and head strides in elements
 * (multiples of 8), 16-byte aligned; the slots of the head-interleaved projections
 * [len, batch, heads, 3 | 2, head_dim] qualify. Every sequence has len_q queries.
 * key_padding_mask: NULL, or uint8 [batch, len_k], 1 = masked, any pattern. A query whose keys are
 * all masked has out = 0 and softmax_lse = -inf (the reference's softmax yields NaN there).
 * key_info: with a mask, device workspace of nmtg_flash_attn_key_info_bytes(batch, len_k) bytes,
 * 4-byte aligned; a small kernel ahead of the others writes each sequence's last live key,
 * which 64-key tiles hold masked keys in front of it, and the mask of those tiles packed to bits
 * (the attention kernels read the packed words, not the mask).
 * time_mask: NULL, or uint8 [len_q, len_k], 1 = masked, shared by every sequence and head (the
 * reference's use_time_mask form; any pattern, a causal one included); not together with
 * key_padding_mask. time_info: with it, device workspace of
 * nmtg_flash_attn_time_info_bytes(len_q, len_k) bytes, 4-byte aligned: a small kernel classifies
 * the mask by patches of 32 x 64 (no masked element / some / all) for both kernel orientations, the
 * attention kernels stop at the last key tile (start at the first query tile) with a live element;
 * the same kernel packs the mask to bits in both orientations (len_q * len_k / 4 bytes), and the
 * attention kernels read one packed word per lane in patches that hold masked elements.
 * causal, dropout_*, seed, offset, softmax_lse [batch, heads, len_q], softmax_d: as above, with
 * max_seqlen_* = len_*.
 * nmtg_flash_attn_batched_bwd: dout has the strides of out; dq, dk, dv have the strides of q, k, v
 * and are written whole (zeros at masked keys). Deterministic: no atomics.
 * ------------------------------------------------------------------------------------------ */
int64_t nmtg_flash_attn_key_info_bytes(int64_t batch, int64_t len_k);

int64_t nmtg_flash_attn_time_info_bytes(int64_t len_q, int64_t len_k);

int nmtg_flash_attn_batched_fwd(const void* q, const void* k, const void* v, void* out,
                                const uint8_t* key_padding_mask, void* key_info,
                                const uint8_t* time_mask, void* time_info, float* softmax_lse,
                                int64_t batch, int64_t heads, int64_t head_dim, int64_t len_q,
                                int64_t len_k, int64_t q_stride_t, int64_t q_stride_b,
                                int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_b,
                                int64_t k_stride_h, int64_t v_stride_t, int64_t v_stride_b,
                                int64_t v_stride_h, int64_t out_stride_t, int64_t out_stride_b,
                                int64_t out_stride_h, float softmax_scale, int causal,
                                int dropout_mode, float dropout_p, const uint8_t* dropout_mask,
                                uint8_t* dropout_mask_out, void* dropout_bits, uint64_t seed,
                                uint64_t offset, int dtype, void* stream);

int nmtg_flash_attn_batched_bwd(const void* dout, const void* q, const void* k, const void* v,
                                const void* out, const float* softmax_lse, void* dq, void* dk,
                                void* dv, float* softmax_d, const uint8_t* key_padding_mask,
                                void* key_info, const uint8_t* time_mask, void* time_info,
                                int64_t batch, int64_t heads, int64_t head_dim,
                                int64_t len_q, int64_t len_k, int64_t q_stride_t, int64_t q_stride_b,
                                int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_b,
                                int64_t k_stride_h, int64_t v_stride_t, int64_t v_stride_b,
                                int64_t v_stride_h, int64_t out_stride_t, int64_t out_stride_b,
                                int64_t out_stride_h, float softmax_scale, int causal,
                                int dropout_mode, float dropout_p, const uint8_t* dropout_mask,
                                void* dropout_bits, int dropout_bits_ready, uint64_t seed,
                                uint64_t offset, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Attention of ONE new query position over cached keys / values (incremental decoding).
 * Reference: the incremental branches of SelfAttnFunc (onmt/modules/optimized/
 *   self_attention_func.py:162-174, one query row against the concatenated cache) and of
 *   EncdecAttnBiasFunc (encdec_attention_func_bias.py:181-213, cached encoder keys / values),
 *   run there as one-row batched GEMMs and a softmax.
 * q [batch, heads * head_dim] (row stride q_stride_b); keys, values: element (t, b, h, d) at
 * t * stride_t + b * stride_b + h * head_dim + d (the reference's time-first cache [Tk, B, E] has
 * stride_t = B * E, stride_b = E); key_mask [batch, tk] (1 = masked key) or NULL.
 * probs [batch * heads, tk] = softmax(round(scale * q . k)) in the tensors' 16-bit type (rows without
 * a live key: zeros), context [batch, heads * head_dim] (row stride ctx_stride_b) = probs x values.
 * Keys and values behind a sentence's last unmasked key are not read (what the cache holds there,
 * NaN included, does not reach the results; the reference's 0 x NaN would).
 * head_dim 32, 64 or 128; tk <= 16384; fp16 / bf16; strides multiples of 8 elements.
 * ------------------------------------------------------------------------------------------ */
int nmtg_attn_decode(const void* q, int64_t q_stride_b, const void* keys, int64_t k_stride_t,
                     int64_t k_stride_b, const void* values, int64_t v_stride_t, int64_t v_stride_b,
                     const uint8_t* key_mask, void* probs, void* context, int64_t ctx_stride_b,
                     int64_t batch, int64_t heads, int64_t head_dim, int64_t tk, float scale,
                     int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Gated feed-forward activation with dropout.
 * Reference: the gated branch of PositionWiseFeedForward.forward, PyTorch ops there
 *   (onmt/modules/optimized/feed_forward.py:188-200), and variational_dropout
 *   (onmt/modules/dropout.py:32-48).
 * x [rows, 2 * inner] (row pitch ld_x elements): a = x[:, :inner], b = x[:, inner:];
 *   act = an nmtg_act code: y = act(a) * b;   act = 5: y = a * sigmoid(b)  (F.glu);
 * then y <- y * keep / (1 - p). dropout_mode 0 none, 1 read `mask`, 2 draw it from Philox
 * (element index row * inner + j, as the other dropout kernels) and store it. mask is uint8
 * [mask_rows, inner]; row m uses mask row m % mask_rows: mask_rows == rows is ordinary dropout,
 * mask_rows == batch over a [time, batch, inner] tensor the reference's variational dropout.
 * y [rows, inner] dense. nmtg_glu_bwd: grad_x [rows, 2 * inner] (pitch ld_grad_x) from grad_y.
 * ------------------------------------------------------------------------------------------ */
int nmtg_glu_fwd(const void* x, int64_t ld_x, void* y, uint8_t* mask, int64_t mask_rows,
                 int64_t rows, int64_t inner, int act, int dropout_mode, float p, uint64_t seed,
                 uint64_t offset, int dtype, void* stream);

int nmtg_glu_bwd(const void* grad_y, const void* x, int64_t ld_x, const uint8_t* mask,
                 int64_t mask_rows, void* grad_x, int64_t ld_grad_x, int64_t rows, int64_t inner,
                 int act, int dropout_mode, float p, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Column sums of a row-major matrix: out[c] = sum_r x[r * ld + c], fp32 accumulation in a fixed
 * order (partial sums per block of rows, then one sum over the partials), result in the dtype
 * of x. The bias gradients of the reference's linear layers: torch.sum(grads, 0)
 * (onmt/modules/optimized/relative_self_attention_func.py:562-563, :715) and the bias gradient
 * of linear_blaslt.backward (onmt/modules/extensions/mlp_blaslt/linear.cpp:59-104).
 * workspace: fp32 scratch of nmtg_colsum_workspace_bytes(rows, cols) bytes. rows, cols < 2^31.
 * ------------------------------------------------------------------------------------------ */
int64_t nmtg_colsum_workspace_bytes(int64_t rows, int64_t cols);

int nmtg_colsum(const void* x, int64_t rows, int64_t cols, int64_t ld, void* out, void* workspace,
                int64_t workspace_bytes, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Elementwise pieces of self-attention with relative position encodings (Transformer-XL form).
 * Reference: RelativeShift.forward / backward and the bias additions and the sum of the two score
 *   terms in RelativeSelfAttnFunc (onmt/modules/optimized/relative_self_attention_func.py:26-76,
 *   :210-217, :246-253, :621-630); the products around them are nmtg_gemm calls.
 *
 * nmtg_rel_query_bias: rw_q[r][d] = q[r * ld_q + d] + r_w_bias[(r % heads) * head_dim + d] and
 *   rr_q likewise with r_r_bias, for r < rows (rows = len_q * batch * heads: the queries as they
 *   lie inside the in-projection output, ld_q = 3 * head_dim there), d < head_dim. rw_q, rr_q
 *   dense [rows, head_dim]. The sums are rounded once to the dtype, as an elementwise add does.
 *
 * nmtg_rel_shift_add: scores[b][i][j] += shift(bd)[b][i][j] for j < len_k, in place, where
 *   shift views bd[b] (dense [len_q, len_r], len_r >= len_k) with a zero column in front as
 *   [len_r + 1, len_q], drops the first row and reads the rest as [len_q, len_r]: with
 *   p = i * len_r + j + len_q, i2 = p / (len_r + 1), c = p % (len_r + 1) the value is 0 if c == 0
 *   and bd[b][i2][c - 1] otherwise.
 *
 * nmtg_rel_shift_bwd: the adjoint, grad_bd[b][i2][c - 1] = grad_scores[b][i][j] at the same
 *   correspondence (0 where j >= len_k or where p < len_q); grad_bd dense [batch, len_q, len_r].
 *
 * nmtg_add_rows: out[r][c] = a[r][c] + b[r][c] for r < rows, c < cols, each matrix with its own row
 *   pitch; out may be a or b. The reference's elementwise sums of two gradient or score terms
 *   (queries_grads.add_(queries_grads_bd), :678; the beta = 1 accumulation of the position scores
 *   of learnable positions into matmul_ac, :264).
 * dtype: NMTG_F16, NMTG_BF16 or NMTG_F32.
 * ------------------------------------------------------------------------------------------ */
int nmtg_rel_query_bias(const void* q, int64_t ld_q, const void* r_w_bias, const void* r_r_bias,
                        void* rw_q, void* rr_q, int64_t rows, int64_t heads, int64_t head_dim,
                        int dtype, void* stream);

int nmtg_rel_shift_add(void* scores, const void* bd, int64_t batch, int64_t len_q, int64_t len_k,
                       int64_t len_r, int dtype, void* stream);

int nmtg_rel_shift_bwd(const void* grad_scores, void* grad_bd, int64_t batch, int64_t len_q,
                       int64_t len_k, int64_t len_r, int dtype, void* stream);

int nmtg_add_rows(void* out, int64_t ld_out, const void* a, int64_t ld_a, const void* b, int64_t ld_b,
                  int64_t rows, int64_t cols, int dtype, void* stream);

/* The relative shift folded into the softmax kernels, so that the score tensor is not passed over once more on either
 * side (reference: the same lines as above plus the softmax + dropout between them,
 * relative_self_attention_func.py:246-300 and :560-630; softmax_apex.h as for nmtg_softmax_dropout_*).
 *
 * nmtg_rel_softmax_dropout_fwd: scores [batch, len_q, len_k] holds the content term on entry; on return it holds
 *   content + shift(bd)[:, :, :len_k] (bd dense [batch, len_q, len_r]; the sum rounded to the dtype as
 *   nmtg_rel_shift_add rounds it), which the backward recomputes the probabilities from, and dropped_out
 *   [batch, len_q, len_k] holds dropout(softmax(masked sum)). key_mask / mask_kind / heads / dropout_mask /
 *   dropout_mode / p / seed / offset as for nmtg_softmax_dropout_fwd with rows = batch * len_q, cols = len_k,
 *   q_len = len_q.
 * nmtg_rel_softmax_dropout_bwd: grad_scores [batch, len_q, len_k] = softmax-dropout backward from the saved summed
 *   scores (as nmtg_softmax_dropout_bwd with saved_is_scores = 1), and grad_bd [batch, len_q, len_r] = the shift's
 *   adjoint of grad_scores (as nmtg_rel_shift_bwd), every element written.
 * Both need len_k a multiple of 16 bytes of elements, 16-byte aligned tensors, len_r >= len_k, at most 4096 keys
 * (2048 in fp32), len_q * (len_r + 1) < 2^31 and batch * len_q < 2^31; other shapes go through the separate calls.
 * dtype: NMTG_F16, NMTG_BF16 or NMTG_F32. */
int nmtg_rel_softmax_dropout_fwd(void* scores, const void* bd, int64_t len_r, const uint8_t* key_mask,
                                 int mask_kind, void* dropped_out, uint8_t* dropout_mask, int dropout_mode,
                                 float p, uint64_t seed, uint64_t offset, int64_t batch, int64_t len_q,
                                 int64_t len_k, int64_t heads, int dtype, void* stream);

int nmtg_rel_softmax_dropout_bwd(const void* grad_dropped, const void* scores, const uint8_t* key_mask,
                                 int mask_kind, const uint8_t* dropout_mask, int dropout_mode, float p,
                                 void* grad_scores, void* grad_bd, int64_t len_r, int64_t batch,
                                 int64_t len_q, int64_t len_k, int64_t heads, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Optimizer-side passes over a list of tensors (one launch per 48 tensors instead of one per tensor).
 * Reference: fused_optim.multi_tensor_adam / multi_tensor_scale / multi_tensor_axpby / multi_tensor_l2norm /
 *   multi_tensor_l2norm_scale
 *   (onmt/modules/extensions/fused_optim/frontend.cpp:45-53; multi_tensor_adam.cu:22-171,
 *   multi_tensor_scale_kernel.cu:29-136, multi_tensor_l2norm_kernel.cu:27-232, :293-367), driven by
 *   FusedAdam.step (onmt/modules/optimized/fused_adam.py:113-191).
 * The lists are HOST arrays of n_tensors device pointers; sizes[t] is tensor t's element count (each
 * tensor dense). fp32 arithmetic whatever the storage type.
 *
 * nmtg_multi_tensor_adam: per element, with g, p, m, v of grads / params / exp_avg / exp_avg_sq:
 *   mode 0 (L2): g += weight_decay * p;  m = beta1 m + (1 - beta1) g;  v = beta2 v + (1 - beta2) g g;
 *   update = (m / c1) / (sqrt(v / c2) + eps), mode 1 (decoupled decay): update += weight_decay * p;
 *   p -= lr * update;  c1 = 1 - beta1^step, c2 = 1 - beta2^step, or 1 without bias_correction.
 *   p, m, v are updated in place; the four lists share one dtype.
 * nmtg_multi_tensor_scale: out = in * scale (dtypes may differ); *noop_flag (device int, may be NULL)
 *   is set to 1 if any input element is inf or NaN, and left alone otherwise.
 * nmtg_multi_tensor_axpby: out = a x + b y; y and out share out_dtype; the flag is raised for inf / NaN
 *   in x (arg_to_check 0), y (1) or either (-1) (multi_tensor_axpby_kernel.cu:27-126).
 * nmtg_multi_tensor_l2norm: norm[0] = sqrt(sum over all tensors of x^2); per_tensor[t] (may be NULL)
 *   = the norm of tensor t; both fp32 on the device; deterministic (fixed-order sums). workspace: fp32
 *   scratch of nmtg_multi_tensor_l2norm_workspace_bytes(n_tensors, sizes) bytes.
 * nmtg_multi_tensor_l2norm_scale: the same norms of `in` (unscaled) while writing out = in * scale in
 *   the same pass (multi_tensor_l2norm_scale_kernel.cu:28-125); same workspace.
 * ------------------------------------------------------------------------------------------ */
int nmtg_multi_tensor_adam(int n_tensors, const void* const* grads, void* const* params,
                           void* const* exp_avg, void* const* exp_avg_sq, const int64_t* sizes, float lr,
                           float beta1, float beta2, float eps, int step, int mode, int bias_correction,
                           float weight_decay, int dtype, void* stream);

int nmtg_multi_tensor_scale(int n_tensors, const void* const* in, void* const* out, const int64_t* sizes,
                            float scale, int* noop_flag, int in_dtype, int out_dtype, void* stream);

int nmtg_multi_tensor_axpby(int n_tensors, const void* const* x, const void* const* y, void* const* out,
                            const int64_t* sizes, float a, float b, int arg_to_check, int* noop_flag,
                            int x_dtype, int out_dtype, void* stream);

int64_t nmtg_multi_tensor_l2norm_workspace_bytes(int n_tensors, const int64_t* sizes);

int nmtg_multi_tensor_l2norm(int n_tensors, const void* const* x, const int64_t* sizes, float* norm,
                             float* per_tensor, void* workspace, int64_t workspace_bytes, int dtype,
                             void* stream);

int nmtg_multi_tensor_l2norm_scale(int n_tensors, const void* const* in, void* const* out,
                                   const int64_t* sizes, float scale, float* norm, float* per_tensor,
                                   void* workspace, int64_t workspace_bytes, int in_dtype, int out_dtype,
                                   void* stream);

/* ------------------------------------------------------------------------------------------
 * Per-kernel timing for benchmarks (no counterpart in the reference, whose tests time whole ops
 * with CUDA events, e.g. onmt/modules/test_layer_norm.py:14-31). Between nmtg_trace_begin() and
 * nmtg_trace_end() every kernel the library enqueues is bracketed by two HIP events on its
 * stream. nmtg_trace_end waits for them and writes lines "name launches total_ms\n" into `out`
 * (NUL-terminated, truncated to `capacity`); it returns the full text length. Not for use while
 * a stream is being captured into a graph. Process-wide switch.
 * ------------------------------------------------------------------------------------------ */
int nmtg_trace_begin(void);
int64_t nmtg_trace_end(char* out, int64_t capacity);

/* ------------------------------------------------------------------------------------------
 * Streaming probes (no counterpart in the reference; a measurement aid like the tracing above).
 * One launch of the simplest kernel with the access mix of the library's bandwidth-bound
 * kernels, to be timed: what this HBM gives such a mix is the practical ceiling their roofline
 * fractions are read against. `bytes` (a multiple of 16) is the size of each buffer.
 *   mode 0  out[i] = a[i]                         one stream read, one written
 *   mode 1  out[i] = a[i] + b[i] (fp32 lanes)     two streams read, one written
 *   mode 2  out[block] = sum of the block's chunk of a (fp32)   read only; `out` holds
 *           nmtg_stream_probe_blocks(bytes) floats
 * ------------------------------------------------------------------------------------------ */
int64_t nmtg_stream_probe_blocks(int64_t bytes);
int nmtg_stream_probe(const void* a, const void* b, void* out, int64_t bytes, int mode, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NMTG_HIP_H_ */
