/*
 * oslo_hip.h -- C ABI of liboslo_hip.so: the fused non-GEMM transformer-layer
 * kernels (LayerNorm / RMSNorm, scaled causal / padding-masked softmax,
 * bias-GeLU, bias-dropout-add; forward and backward) for AMD gfx950.
 *
 * Conventions shared by every entry point
 *   - All tensor arguments are raw DEVICE pointers to contiguous row-major
 *     storage.  The library never allocates, frees or synchronises: the caller
 *     owns every output and every workspace (sizes from oslo_workspace_bytes).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Launches are asynchronous on that stream.
 *   - Return value: OSLO_OK (0) or a negative OSLO_ERR_* code; the message
 *     for the calling thread's last failure is oslo_hip_last_error().
 *   - dtype arguments take OSLO_DTYPE_* values.  Accumulation is fp32.
 *   - Element counts are 64-bit; a tensor may exceed 2^31 elements, and a
 *     softmax may have more than 2^31 rows.  A GPU dispatch holds fewer than
 *     2^32 work-items: an entry point whose problem needs more issues several
 *     launches on the stream (still without synchronising).
 *
 * Each declaration cites the interface of the reference (EleutherAI/oslo) it
 * replaces; paths are relative to the reference's repository root.
 */
#ifndef OSLO_HIP_H
#define OSLO_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OSLO_HIP_ABI_VERSION 1

#define OSLO_OK 0
#define OSLO_ERR_INVALID_ARGUMENT (-1)
#define OSLO_ERR_UNSUPPORTED (-2)
#define OSLO_ERR_WORKSPACE (-3)
#define OSLO_ERR_LAUNCH (-4)

#define OSLO_DTYPE_F32 0
#define OSLO_DTYPE_F16 1
#define OSLO_DTYPE_BF16 2
#define OSLO_DTYPE_F64 3 /* LayerNorm / RMSNorm entry points only */

/* ops for oslo_workspace_bytes */
#define OSLO_OP_LN_BWD 1
#define OSLO_OP_RMS_BWD 2
#define OSLO_OP_BIAS_GELU_BWD 3
#define OSLO_OP_BIAS_DROPOUT_ADD_BWD 4
#define OSLO_OP_BIAS_DROPOUT_ADD_NORM_BWD 5

/* ---- library state ----------------------------------------------------- */

/* Message of the calling thread's most recent failing call ("" if none). */
const char *oslo_hip_last_error(void);
/* Architecture the device code was compiled for ("gfx950"). */
const char *oslo_hip_arch(void);
int oslo_hip_abi_version(void);

/* Bytes of fp32 scratch the backward entry point `op` needs for an
 * [n1, n2] problem (column-partial sums for the parameter gradients).
 * Replaces the part_grad_gamma / part_grad_beta allocation inside
 * oslo/torch/_C/csrc/fused_layer_norm.cu:831-833, moved to the caller. */
int64_t oslo_workspace_bytes(int op, int64_t n1, int64_t n2);

/* ---- LayerNorm / RMSNorm ----------------------------------------------- *
 * x is [n1, n2] of dtype_in; y, gamma, beta have dtype_out; mean / invvar are
 * fp32 [n1].  Allowed (dtype_in, dtype_out): (f32,f32) (f32,f16) (f32,bf16)
 * (f16,f16) (bf16,bf16) (f64,f64) -- the matrix of
 * oslo/torch/_C/csrc/includes/type_shim.h:128-237.  For (f64,f64) every
 * tensor, mean and invvar included, is double and accumulation is double
 * (type_shim.h:172-186: U = double); the workspace is not used.  That pair is
 * a plain two-pass kernel meant for checking, not for throughput.
 * gamma == NULL (then beta must be NULL too) selects the non-affine form.  */

/* Replaces layer_norm_forward, layer_norm_forward_affine and
 * layer_norm_forward_affine_mixed_dtypes
 * (oslo/torch/_C/csrc/FusedLayerNormBinder.cpp:135-207, 404-417 ->
 * cuda_layer_norm, fused_layer_norm.cu:771-788).
 * y = (x - mean) * invvar * gamma + beta evaluated in fp32, rounded once.  */
int oslo_ln_fwd(const void *x, const void *gamma, const void *beta, void *y,
                void *mean, void *invvar, int64_t n1, int64_t n2, double eps,
                int dtype_in, int dtype_out, void *stream);

/* Replaces layer_norm_backward and layer_norm_backward_affine
 * (FusedLayerNormBinder.cpp:221-266 -> cuda_layer_norm_gradient,
 * fused_layer_norm.cu:908-935; three launches there, one pass + a finalize
 * here).  dy, gamma, dgamma, dbeta have dtype_out; x, dx have dtype_in.
 * dgamma / dbeta may be NULL only when gamma is NULL.                      */
int oslo_ln_bwd(const void *dy, const void *x, const void *mean,
                const void *invvar, const void *gamma, void *dx, void *dgamma,
                void *dbeta, void *workspace, int64_t workspace_bytes,
                int64_t n1, int64_t n2, int dtype_in, int dtype_out,
                void *stream);

/* oslo_ln_bwd without a workspace argument and without any allocation.  It
 * has no counterpart in the reference; it is for callers that cannot
 * allocate device memory around the call: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  The fp32 partial
 * rows of dgamma / dbeta go to an array of
 * OSLO_LN_BWD_STATIC_SCRATCH_BYTES bytes that is part of the library's device
 * code (each GPU the library runs on holds its copy until the process ends).
 * A problem whose oslo_workspace_bytes(OSLO_OP_LN_BWD, n1, n2) exceeds that
 * size is refused with OSLO_ERR_WORKSPACE (n2 up to 8192 fits at any n1 on a
 * 256-CU part).  Results equal oslo_ln_bwd's bit for bit.  All calls on one
 * GPU share the array: calls that may overlap there (different streams or
 * host threads without ordering between them) race and must use oslo_ln_bwd
 * with their own workspaces instead.                                        */
#define OSLO_LN_BWD_STATIC_SCRATCH_BYTES (16 * 1024 * 1024)
int oslo_ln_bwd_static(const void *dy, const void *x, const void *mean,
                       const void *invvar, const void *gamma, void *dx,
                       void *dgamma, void *dbeta, int64_t n1, int64_t n2,
                       int dtype_in, int dtype_out, void *stream);

/* Replaces rms_norm_forward, rms_norm_forward_affine and
 * rms_norm_forward_affine_mixed_dtypes (FusedLayerNormBinder.cpp:285-358 ->
 * cuda_rms_norm, fused_layer_norm.cu:790-806).
 * y = gamma * round_out(x * invvar): the normalised value is rounded to
 * dtype_out before the scale, as fused_layer_norm.cu:338 and
 * oslo/torch/nn/modules/layer_norm.py:27-30 both do.                       */
int oslo_rms_fwd(const void *x, const void *gamma, void *y, void *invvar,
                 int64_t n1, int64_t n2, double eps, int dtype_in,
                 int dtype_out, void *stream);

/* Replaces rms_norm_backward and rms_norm_backward_affine
 * (FusedLayerNormBinder.cpp:360-402 -> cuda_rms_norm_gradient,
 * fused_layer_norm.cu:937-963).                                            */
int oslo_rms_bwd(const void *dy, const void *x, const void *invvar,
                 const void *gamma, void *dx, void *dgamma, void *workspace,
                 int64_t workspace_bytes, int64_t n1, int64_t n2, int dtype_in,
                 int dtype_out, void *stream);

/* ---- scaled masked softmax --------------------------------------------- *
 * Input, output and gradients share one dtype (f32, f16 or bf16).          */

/* Replaces fused_scaled_upper_triang_masked_softmax_forward
 * (oslo/torch/_C/csrc/FusedScaleMaskSoftmaxBinder.cpp:76-86, 122-124; the
 * reference declares fwd_cuda but ships no definition).  x, y are
 * [attn_batches, sq, sk]; key j of query i is visible when
 * j <= i + (sk - sq); y = softmax(scale * x) over the visible keys, exact 0
 * elsewhere -- the semantics of
 * oslo/transformers/models/gpt2/modeling_gpt2.py:116-138.                  */
int oslo_softmax_causal_fwd(const void *x, void *y, int64_t attn_batches,
                            int64_t sq, int64_t sk, float scale, int dtype,
                            void *stream);

/* Replaces fused_scaled_upper_triang_masked_softmax_backward
 * (FusedScaleMaskSoftmaxBinder.cpp:88-105, 125-127).
 * dx = scale * y * (dy - sum_j dy_j y_j).  dx may alias dy.                */
int oslo_softmax_causal_bwd(const void *dy, const void *y, void *dx,
                            int64_t attn_batches, int64_t sq, int64_t sk,
                            float scale, int dtype, void *stream);

/* Replaces fused_scaled_masked_softmax_forward
 * (FusedScaleMaskSoftmaxBinder.cpp:39-49, 112-114).  x, y are
 * [b, np, sq, sk]; mask is uint8/bool [mask_b, 1, mask_sq, sk] with
 * mask_b in {1, b} and mask_sq in {1, sq}; non-zero = masked out.  Masked
 * keys get probability exactly 0 (the limit of the additive -10000 of
 * oslo/transformers/models/bert/modeling_bert.py:298-306 and
 * modeling_gpt2.py:573-581); a row whose keys are all masked becomes the
 * uniform 1/sk that masked_fill(mask, -10000) followed by softmax gives.   */
int oslo_softmax_masked_fwd(const void *x, const uint8_t *mask, void *y,
                            int64_t b, int64_t np, int64_t sq, int64_t sk,
                            int64_t mask_b, int64_t mask_sq, float scale,
                            int dtype, void *stream);

/* Replaces fused_scaled_masked_softmax_backward
 * (FusedScaleMaskSoftmaxBinder.cpp:51-64, 115-117).  mask may be NULL (the
 * reference signature has none); when given, loads of masked keys are
 * skipped, which is valid because y is exactly 0 there unless the whole row
 * is masked (such rows are then read in full).  dx may alias dy.           */
int oslo_softmax_masked_bwd(const void *dy, const void *y, const uint8_t *mask,
                            void *dx, int64_t b, int64_t np, int64_t sq,
                            int64_t sk, int64_t mask_b, int64_t mask_sq,
                            float scale, int dtype, void *stream);

/* Causal mask and padding mask in one call: the attention of a causal model
 * that is run on padded batches.  The reference applies both,
 * torch.where(causal, w, -1e4) followed by "+ attention_mask"
 * (oslo/transformers/models/gpt2/modeling_gpt2.py:126-136, mask built at
 * :573-581); its softmax shim has no entry point for the combination.  Same
 * arguments as oslo_softmax_masked_fwd / _bwd; key j of query i is hidden when
 * the mask says so OR j > i + (sk - sq).  Loads stop at the diagonal as in
 * oslo_softmax_causal_fwd, and mask bytes beyond it are not read.  Hidden
 * keys get probability exactly 0; a row without any visible key (a fully
 * padded sample, left padding) becomes the uniform 1/sk, as in
 * oslo_softmax_masked_fwd.  In the backward entry point mask may be NULL.   */
int oslo_softmax_causal_masked_fwd(const void *x, const uint8_t *mask, void *y,
                                   int64_t b, int64_t np, int64_t sq,
                                   int64_t sk, int64_t mask_b, int64_t mask_sq,
                                   float scale, int dtype, void *stream);
int oslo_softmax_causal_masked_bwd(const void *dy, const void *y,
                                   const uint8_t *mask, void *dx, int64_t b,
                                   int64_t np, int64_t sq, int64_t sk,
                                   int64_t mask_b, int64_t mask_sq, float scale,
                                   int dtype, void *stream);

/* Replaces get_batch_per_block (FusedScaleMaskSoftmaxBinder.cpp:66-70,
 * 118-121): softmax rows one workgroup of the masked kernel handles.  The
 * kernels here have no divisibility requirement on it.  Negative on error. */
int oslo_softmax_batch_per_block(int64_t sq, int64_t sk, int64_t b,
                                 int64_t np);

/* ---- softmax with the attention-probability dropout fused in ------------ *
 * Replaces the pair softmax -> attn_dropout that follows the scores in
 * oslo/transformers/models/gpt2/modeling_gpt2.py:138-142 (causal) and
 * oslo/transformers/models/bert/modeling_bert.py:306-310 (padding mask):
 *   out = keep * softmax(mask(scale * x)) / (1 - p).
 * The keep decisions are the Philox stream of oslo_philox_mask over the
 * flattened output (element i = row * sk + key: group i >> 3, bit i & 7), so
 * nothing but the row statistics is stored for the backward pass:
 * stats is float [rows][2] = {max_j of scale * log2(e) * x_j over the visible
 * keys, 1 / sum_j exp2(scale * log2(e) * x_j - max)}, or {0, -1/sk} for a row
 * without a visible key.  The backward pass takes the saved *input* x (not
 * the output), recomputes the probabilities y from x and stats, regenerates
 * the keep bits from the same (p, seed, offset) and returns
 *   dx = scale * y * (dp - sum_k dp_k y_k),  dp = keep * dout / (1 - p).
 * With p == 0 the forward output equals oslo_softmax_*_fwd bit for bit.
 * dx may alias dout or x.  Shapes and mask rules as for the entry points
 * above; advance the generator offset by 4 per call.                        */
int oslo_softmax_causal_dropout_fwd(const void *x, void *out, float *stats,
                                    int64_t attn_batches, int64_t sq,
                                    int64_t sk, float scale, float p,
                                    uint64_t seed, uint64_t offset, int dtype,
                                    void *stream);
int oslo_softmax_causal_dropout_bwd(const void *dout, const void *x,
                                    const float *stats, void *dx,
                                    int64_t attn_batches, int64_t sq,
                                    int64_t sk, float scale, float p,
                                    uint64_t seed, uint64_t offset, int dtype,
                                    void *stream);
int oslo_softmax_masked_dropout_fwd(const void *x, const uint8_t *mask,
                                    void *out, float *stats, int64_t b,
                                    int64_t np, int64_t sq, int64_t sk,
                                    int64_t mask_b, int64_t mask_sq,
                                    float scale, float p, uint64_t seed,
                                    uint64_t offset, int dtype, void *stream);
int oslo_softmax_masked_dropout_bwd(const void *dout, const void *x,
                                    const uint8_t *mask, const float *stats,
                                    void *dx, int64_t b, int64_t np, int64_t sq,
                                    int64_t sk, int64_t mask_b, int64_t mask_sq,
                                    float scale, float p, uint64_t seed,
                                    uint64_t offset, int dtype, void *stream);

/* The same pair for the causal + padding mask combination
 * (oslo_softmax_causal_masked_fwd above).                                   */
int oslo_softmax_causal_masked_dropout_fwd(const void *x, const uint8_t *mask,
                                           void *out, float *stats, int64_t b,
                                           int64_t np, int64_t sq, int64_t sk,
                                           int64_t mask_b, int64_t mask_sq,
                                           float scale, float p, uint64_t seed,
                                           uint64_t offset, int dtype,
                                           void *stream);
int oslo_softmax_causal_masked_dropout_bwd(const void *dout, const void *x,
                                           const uint8_t *mask,
                                           const float *stats, void *dx,
                                           int64_t b, int64_t np, int64_t sq,
                                           int64_t sk, int64_t mask_b,
                                           int64_t mask_sq, float scale, float p,
                                           uint64_t seed, uint64_t offset,
                                           int dtype, void *stream);

/* ---- softmax with an additive floating-point term ------------------------ *
 * y = softmax(scale * x + M) -- the form in which the reference's models
 * mask and bias their scores: `attention_scores + attention_mask` with the
 * [b, 1, 1, sk] term (1 - m) * -10000
 * (oslo/transformers/models/bert/modeling_bert.py:298-306,
 * oslo/transformers/models/gpt2/modeling_gpt2.py:136 with the mask built at
 * :573-581), the finfo.min fill of
 * oslo/transformers/models/bart/modeling_bart.py:123-136, 262-284, the
 * relative-position bias [1, np, sq, sk] of
 * oslo/transformers/models/t5/modeling_t5.py:508-514, and LightSeq's additive
 * [batch, to_len] mask (oslo/lightseq2/csrc/kernels/cuda/softmax_kernels.cu:
 * 35-127).  The reference has no fused entry point for it.
 *
 * x, y are [b, np, sq, sk].  M ("bias") has the dtype bias_dtype = dtype or
 * OSLO_DTYPE_F32 and is addressed as
 *   M[bi * bias_stride_b + hi * bias_stride_h + qi * bias_stride_q + key]
 * (strides in elements, 0 = that dimension is broadcast; keys contiguous).
 * The sum is one fused multiply-add in float, so the additive semantics are
 * those of a float evaluation of the unfused chain: a row whose terms are all
 * -10000 gives softmax(scale * x), a row whose terms are all the lowest
 * finite value gives the uniform distribution (the term absorbs the logit),
 * a row whose terms are all -inf gives NaN, as torch.softmax does.
 * flags: OSLO_SOFTMAX_CAUSAL hides key j of query i when j > i + (sk - sq)
 * as well (exact zeros, also in a query row that the diagonal leaves without
 * any key when sq > sk; neither x nor M is read there);
 * OSLO_SOFTMAX_SKIP_HIDDEN reads M first and leaves the logits of a 16-byte
 * chunk unread when every term of it is at or below the lowest finite
 * bfloat16 (-3.39e38; the lowest float and -inf are), where the float sum is
 * the term itself whatever the logit (below 1e30 in magnitude): worth it
 * when M is small (a broadcast mask), not for a dense bias.
 * The backward pass is that of every softmax,
 *   dx = scale * y * (dy - sum_j dy_j y_j),
 * and takes M (may be NULL) only to skip loads under the same flag: y is
 * exactly 0 where the term absorbs the logit, unless the whole row is like
 * that (such rows are read in full).  dx may alias dy.  The gradient with
 * respect to M is dx / scale summed over the broadcast dimensions; it is left
 * to the caller.                                                            */
#define OSLO_SOFTMAX_CAUSAL 1
#define OSLO_SOFTMAX_SKIP_HIDDEN 2
int oslo_softmax_bias_fwd(const void *x, const void *bias, void *y, int64_t b,
                          int64_t np, int64_t sq, int64_t sk,
                          int64_t bias_stride_b, int64_t bias_stride_h,
                          int64_t bias_stride_q, int bias_dtype, int flags,
                          float scale, int dtype, void *stream);
int oslo_softmax_bias_bwd(const void *dy, const void *y, const void *bias,
                          void *dx, int64_t b, int64_t np, int64_t sq,
                          int64_t sk, int64_t bias_stride_b,
                          int64_t bias_stride_h, int64_t bias_stride_q,
                          int bias_dtype, int flags, float scale, int dtype,
                          void *stream);

/* The same with the attention-probability dropout fused in (see the dropout
 * entry points above): stats is float [rows][2] = {max_j (scale * x_j + M_j),
 * 1 / sum_j exp(scale * x_j + M_j - max)}; the backward pass takes x, M and
 * stats and recomputes the probabilities.                                   */
int oslo_softmax_bias_dropout_fwd(const void *x, const void *bias, void *out,
                                  float *stats, int64_t b, int64_t np,
                                  int64_t sq, int64_t sk, int64_t bias_stride_b,
                                  int64_t bias_stride_h, int64_t bias_stride_q,
                                  int bias_dtype, int flags, float scale,
                                  float p, uint64_t seed, uint64_t offset,
                                  int dtype, void *stream);
int oslo_softmax_bias_dropout_bwd(const void *dout, const void *x,
                                  const void *bias, const float *stats,
                                  void *dx, int64_t b, int64_t np, int64_t sq,
                                  int64_t sk, int64_t bias_stride_b,
                                  int64_t bias_stride_h, int64_t bias_stride_q,
                                  int bias_dtype, int flags, float scale,
                                  float p, uint64_t seed, uint64_t offset,
                                  int dtype, void *stream);

/* ---- dropout state in device memory ------------------------------------- *
 * No counterpart in the reference.  For callers that capture launches in a
 * HIP graph: a (seed, offset) pair passed by value is frozen into the graph
 * and every replay would draw the same mask.  After
 * oslo_rng_from_device(state), the dropout entry points called NEXT ON THE
 * SAME HOST THREAD (bias-dropout-add, its fusion into the norm, softmax with
 * dropout; forward and backward) ignore their `seed` argument and make their
 * kernels read, when they run, seed = state[0] and offset = state[1] + the
 * `offset` argument from device memory.  oslo_rng_from_device(NULL) restores
 * the by-value behaviour.  `state` points to two uint64 in device memory that
 * the caller owns and updates (e.g. state[1] += 4 between calls, in a kernel
 * of its own that is captured too); the setting itself is per host thread
 * and is not part of any graph.                                            */
int oslo_rng_from_device(const uint64_t *state);

/* ---- bias-GeLU (tanh approximation) ------------------------------------ *
 * x, y, g, dx are [rows, cols]; bias, dbias are [cols]; one dtype for all. */

/* Replaces _fused_bias_gelu_fwb / _fused_gelu_fwb
 * (oslo/torch/nn/modules/functional.py:23-25, 37-40), TorchScript there.
 * bias == NULL gives plain GeLU.                                           */
int oslo_bias_gelu_fwd(const void *x, const void *bias, void *y, int64_t rows,
                       int64_t cols, int dtype, void *stream);

/* Replaces _fused_bias_gelu_bwd / _fused_gelu_bwd (functional.py:28-34,
 * 43-50) and the autograd sum-to-size that turns the full-size bias gradient
 * of functional.py:84 into [cols]: dbias = column sum of dx, fused here.
 * dbias may be NULL (then workspace may be NULL).                          */
int oslo_bias_gelu_bwd(const void *g, const void *x, const void *bias,
                       void *dx, void *dbias, void *workspace,
                       int64_t workspace_bytes, int64_t rows, int64_t cols,
                       int dtype, void *stream);

/* ---- bias-dropout-add --------------------------------------------------- *
 * Dropout mask: element i (row-major index) belongs to group i / 8; the
 * group's four 32-bit words are Philox4x32-10 with key = seed and counter =
 * (offset_lo, offset_hi, group_lo, group_hi); element i takes the 16-bit half
 * ((i % 8) & 1) of word (i % 8) / 2 (low half first) and is KEPT when that
 * value >= round(p * 65536).  Kept values are scaled by 1 / (1 - p).
 * The keep probability is therefore 1 - round(p * 65536) / 65536, p rounded
 * to a multiple of 2^-16, while the scale uses p itself: for p = 0.1 an
 * element is kept with probability 0.899994 and the expectation of the
 * output is 7e-6 (relative) below the input's.                              */

/* Replaces fused_bias_dropout (functional.py:295-298:
 * F.dropout(x + bias, p, training)) plus the residual add its callers do
 * next (oslo/transformers/models/gpt2/modeling_gpt2.py:300, 369, 396).
 * out = keep * (x + bias) / (1 - p) + residual.  bias, residual, mask_out may
 * each be NULL; p == 0 (or eval mode: pass p = 0) is the identity mask.
 * mask_out, if given, receives the keep mask as one uint8 per element.     */
int oslo_bias_dropout_add_fwd(const void *x, const void *bias,
                              const void *residual, void *out,
                              uint8_t *mask_out, int64_t rows, int64_t cols,
                              float p, uint64_t seed, uint64_t offset,
                              int dtype, void *stream);

/* Backward of the above: dx = keep * g / (1 - p) with the mask regenerated
 * from (seed, offset); dbias = column sum of dx (NULL to skip); the residual
 * gradient is g itself.  dx may alias g.                                   */
int oslo_bias_dropout_add_bwd(const void *g, void *dx, void *dbias,
                              void *workspace, int64_t workspace_bytes,
                              int64_t rows, int64_t cols, float p,
                              uint64_t seed, uint64_t offset, int dtype,
                              void *stream);

/* ---- bias-dropout-add fused into the following LayerNorm / RMSNorm ------ *
 * Replaces the chain FusedBiasDropout -> residual add -> LayerNorm of the
 * post-LN blocks (oslo/transformers/models/bert/modeling_bert.py:343-346,
 * 446-449: LayerNorm(dropout(dense(x) + bias) + input_tensor)) and the
 * residual add -> ln_2 of the pre-LN blocks (modeling_gpt2.py:369-393):
 *   h = keep * (x + bias) / (1 - p) + residual   (rounded once, as
 *                                                 oslo_bias_dropout_add_fwd)
 *   y = norm(h)                                  (as oslo_ln_fwd / oslo_rms_fwd
 *                                                 of the stored h)
 * One dtype for x, bias, residual, h_out, y, gamma, beta.  bias, residual,
 * gamma/beta and h_out may be NULL; h_out receives h, which the backward
 * pass (and a pre-LN block's next residual) needs.  rms != 0 selects RMSNorm
 * (beta and mean are then ignored).  Keep mask: that of
 * oslo_bias_dropout_add_fwd for the same (p, seed, offset).                 */
int oslo_bias_dropout_add_norm_fwd(const void *x, const void *bias,
                                   const void *residual, const void *gamma,
                                   const void *beta, void *h_out, void *y,
                                   float *mean, float *invvar, int64_t n1,
                                   int64_t n2, double eps, float p,
                                   uint64_t seed, uint64_t offset, int rms,
                                   int dtype, void *stream);

/* Backward of the above in one pass over dy and h (plus a finalize launch):
 *   dh    = norm_backward(dy; h, mean, invvar, gamma) + dh_extra
 *   dres  = dh                      gradient of the residual (and of h)
 *   dx    = keep * dh / (1 - p)     gradient of x; NULL allowed when p == 0,
 *                                   where it equals dres
 *   dbias = column sums of dx as stored; dgamma, dbeta as oslo_ln_bwd.
 * dh_extra (may be NULL) is the gradient that reaches h from its other
 * consumers -- in a pre-LN block h is also the next residual -- the fused
 * residual-gradient add of the reference's
 * oslo/lightseq2/csrc/kernels/cuda/normalize_kernels.cu:608-616.
 * Workspace: oslo_workspace_bytes(OSLO_OP_BIAS_DROPOUT_ADD_NORM_BWD, n1, n2).
 * Outputs must not alias inputs.                                            */
int oslo_bias_dropout_add_norm_bwd(const void *dy, const void *dh_extra,
                                   const void *h, const float *mean,
                                   const float *invvar, const void *gamma,
                                   void *dres, void *dx, void *dgamma,
                                   void *dbeta, void *dbias, void *workspace,
                                   int64_t workspace_bytes, int64_t n1,
                                   int64_t n2, float p, uint64_t seed,
                                   uint64_t offset, int rms, int dtype,
                                   void *stream);

/* ---- multi-tensor Adam / AdamW ----------------------------------------- *
 * Replaces multi_tensor_adam (oslo/torch/_C/csrc/FusedAdamBinder.cpp:1-15 ->
 * multi_tensor_adam_cuda, oslo/torch/_C/csrc/multi_tensor_adam.cu:112-136,
 * functor :22-110), called by FusedAdam.step
 * (oslo/torch/optim/fused_adam.py:96-184).  g, p, m, v are HOST arrays of
 * ntensors device pointers (gradient, parameter, exp_avg, exp_avg_sq of each
 * tensor) and sizes the element counts; all tensors share `dtype` (f32, f16,
 * bf16; the reference dispatches double, float and half), the math is fp32:
 *   mode 0 (L2):    g += decay * p
 *   m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g g
 *   update = (m / bc1) / (sqrt(v / bc2) + eps)  [+ decay * p in mode 1, AdamW]
 *   p -= lr * update
 * with bc1 = 1 - b1^step, bc2 = 1 - b2^step when bias_correction == 1, else
 * 1.  p, m, v are updated in place.  The tensor table travels in kernel
 * arguments (64 tensors per launch); nothing is allocated or copied.  The
 * reference's chunk_size and noop_flag arguments have no effect on its
 * result (the flag test is commented out, multi_tensor_adam.cu:29-31) and
 * are not part of this signature.                                          */
int oslo_multi_tensor_adam(const void *const *g, void *const *p, void *const *m,
                           void *const *v, const int64_t *sizes,
                           int64_t ntensors, float lr, float beta1, float beta2,
                           float eps, int step, int mode, int bias_correction,
                           float weight_decay, int dtype, void *stream);

/* ---- the other multi-tensor optimizer steps and their norms ------------- *
 * Same conventions as oslo_multi_tensor_adam: the list arguments are HOST
 * arrays of ntensors device pointers, sizes the element counts, the math is
 * fp32, nothing is allocated or copied, the tensor table travels in kernel
 * arguments (48 tensors per launch).  Tensors without elements are allowed.  */

/* Replaces multi_tensor_sgd (oslo/torch/_C/csrc/multi_tensor_sgd.cu:124-208,
 * functor :29-122), called by FusedSGD.step (oslo/torch/optim/fused_sgd.py:
 * 268-282).  g, w, mom: gradient, weight, momentum buffer; w_copy (or null): a
 * 16-bit copy of the updated float32 weight (dtype_copy f16 or bf16).
 *   g *= scale;  [g += wd w]  (before the momentum unless wd_after_momentum)
 *   momentum != 0:  mom = first_run ? g : momentum mom + (1 - dampening) g
 *                   g = nesterov ? g + momentum mom : mom
 *   w += -lr g
 * Type combinations: gradients and weights of one type (f32, f16, bf16), or
 * 16-bit gradients with f32 weights (the reference: the four cases of :139-201).
 * mom has the weights' type and is written only when momentum != 0.  When
 * noop_flag (device int, or null) is non-zero the launch changes nothing (:35).  */
int oslo_multi_tensor_sgd(const void *const *g, void *const *w, void *const *mom,
                          void *const *w_copy, const int64_t *sizes, int64_t ntensors,
                          float weight_decay, float momentum, float dampening, float lr,
                          int nesterov, int first_run, int wd_after_momentum, float scale,
                          int dtype_grad, int dtype_weight, int dtype_copy,
                          const int *noop_flag, void *stream);

/* Replaces multi_tensor_adagrad (oslo/torch/_C/csrc/multi_tensor_adagrad.cu:
 * 86-101, functor :24-84), called by FusedAdagrad.step
 * (oslo/torch/optim/fused_adagrad.py:112-131).  g, p, h: gradient, parameter,
 * sum of squares, one dtype.
 *   mode 0 (L2):  g += decay p;  h += g g;  p -= lr g / (sqrt(h) + eps)
 *   mode 1:       h += g g;  p -= lr (g / (sqrt(h) + eps) + decay p)        */
int oslo_multi_tensor_adagrad(const void *const *g, void *const *p, void *const *h,
                              const int64_t *sizes, int64_t ntensors, float lr, float eps,
                              int mode, float weight_decay, int dtype, void *stream);

/* The element-wise part of multi_tensor_novograd (oslo/torch/_C/csrc/
 * multi_tensor_novograd.cu:111-148, functor :30-109), called by
 * FusedNovograd.step (oslo/torch/optim/fused_novograd.py:228-262).
 * grad_norms: device float[ntensors], the blended per-tensor gradient norms
 * (the reference's host function updates them first through
 * multi_tensor_norm_out: call oslo_multi_tensor_norm with blend = 1,
 * alpha = beta2, beta = 1 - beta2 before this).  With
 * denom = grad_norms[t] / bc2 + eps, bc1 = 1 - beta1^step,
 * bc2 = sqrt(1 - beta2^step) (both 1 without bias_correction) and
 * beta3 = grad_averaging ? 1 - beta1 : 1:
 *   moment_mode 0:  g = g / denom + decay p;  m = beta1 m + beta3 g;  p -= lr m / bc1
 *   moment_mode 1:  m = beta1 m + beta3 g;  p -= lr ((m / bc1) / denom + decay p)  */
int oslo_multi_tensor_novograd(const void *const *g, void *const *p, void *const *m,
                               const int64_t *sizes, int64_t ntensors, const float *grad_norms,
                               float lr, float beta1, float beta2, float eps, int step,
                               int bias_correction, float weight_decay, int grad_averaging,
                               int moment_mode, int dtype, void *stream);

/* The two element-wise stages of multi_tensor_lamb (oslo/torch/_C/csrc/
 * multi_tensor_lamb.cu:285-352; stage 1 :41-204, stage 2 :208-283).  The
 * reference's host function runs: per-tensor L2 norms of the parameters,
 * stage 1, per-tensor L2 norms of the updates, stage 2; the norms are
 * oslo_multi_tensor_norm calls.
 * Stage 1 (g, p, m, v; the update direction overwrites g):
 *   g /= clip, clip = *global_grad_norm > max_grad_norm ? ratio of the two : 1
 *   mode 0: g += decay p
 *   m = beta1 m + beta3 g;  v = beta2 v + (1 - beta2) g g
 *   update = (m / bc1) / (sqrt(v / bc2) + eps)  [+ decay p in mode 1]
 * Stage 2 (update, p):  p -= ratio update, ratio = lr * param_norm / update_norm
 * for tensors under weight decay (all tensors with use_nvlamb) when both norms
 * are non-zero, else lr.  global_grad_norm, param_norms, update_norms: device
 * floats.                                                                   */
int oslo_multi_tensor_lamb_stage1(void *const *g, const void *const *p, void *const *m,
                                  void *const *v, const int64_t *sizes, int64_t ntensors,
                                  float beta1, float beta2, float eps, int step,
                                  int bias_correction, float weight_decay, int grad_averaging,
                                  int mode, const float *global_grad_norm, float max_grad_norm,
                                  int dtype, void *stream);
int oslo_multi_tensor_lamb_stage2(const void *const *update, void *const *p,
                                  const int64_t *sizes, int64_t ntensors,
                                  const float *param_norms, const float *update_norms, float lr,
                                  float weight_decay, int use_nvlamb, int dtype, void *stream);

/* Replaces multi_tensor_l2norm (oslo/torch/_C/csrc/multi_tensor_l2norm.cu:
 * 257-317; kernels :29-98, clean-up :174-198) and multi_tensor_norm_out
 * (:323-385; max norm :102-172, clean-up :200-255).  norm_type 2: L2 norm,
 * 0: largest magnitude.  out_global (device float, or null): the norm over all
 * tensors.  out_per_tensor (device float[ntensors], or null): one norm per
 * tensor, written (blend = 0) or blended into the stored value (blend = 1):
 *   L2:  out = sqrt(alpha out^2 + beta sum of squares);  max:  out = alpha out + beta max.
 * partials: workspace of partials_len floats, at least
 * oslo_multi_tensor_norm_partials(sizes, ntensors, dtype); the sums are folded
 * in a fixed order (no atomics).  A partial result that is not finite sets
 * *noop_flag (device int, or null) to 1 (:87-89).  With skip_if_flag the
 * call does nothing (the outputs keep their contents) while *noop_flag is
 * already raised when its kernels start.                                     */
int64_t oslo_multi_tensor_norm_partials(const int64_t *sizes, int64_t ntensors, int dtype);
int oslo_multi_tensor_norm(const void *const *x, const int64_t *sizes, int64_t ntensors,
                           int dtype, float *partials, int64_t partials_len, float *out_global,
                           float *out_per_tensor, int norm_type, int blend, float alpha,
                           float beta, int *noop_flag, int skip_if_flag, void *stream);

/* The two element-wise stages of multi_tensor_lamb_mp (oslo/torch/_C/csrc/
 * multi_tensor_lamb_mp.cu:324-426; stage 1 :40-205, stage 2 :209-322), called
 * by FusedMixedPrecisionLamb.step (oslo/torch/optim/
 * fused_mixed_precision_lamb.py:268-286).  As the plain stages above, except:
 * step (int), lr, max_grad_norm and inv_scale (float) are DEVICE scalars, read
 * when the kernels run, so a training step needs no host synchronisation;
 * the gradient is multiplied by *inv_scale first; the bias corrections
 * 1 - beta^step are formed on the device (in double, then rounded to
 * float, like the host-side ones of the plain stages; the reference forms
 * them with a float power, :54-59); both stages do nothing while
 * *noop_flag (device int, or null) is non-zero.  Stage 1: gradients of
 * dtype_grad, parameters and moments of dtype_param (the same, or f32 master
 * values).  Stage 2: with p_copy (or null) the new f32 parameter is also
 * written in the update's type (the model's 16-bit weights).  The norms of
 * the reference's "mp" host function are oslo_multi_tensor_norm calls with
 * skip_if_flag = 1 (multi_tensor_l2norm_mp.cu:33-35).                        */
int oslo_multi_tensor_lamb_mp_stage1(void *const *g, const void *const *p, void *const *m,
                                     void *const *v, const int64_t *sizes, int64_t ntensors,
                                     float beta1, float beta2, float eps, const int *step,
                                     int bias_correction, float weight_decay,
                                     int grad_averaging, int mode,
                                     const float *global_grad_norm, const float *max_grad_norm,
                                     const float *inv_scale, const int *noop_flag,
                                     int dtype_grad, int dtype_param, void *stream);
int oslo_multi_tensor_lamb_mp_stage2(const void *const *update, void *const *p,
                                     void *const *p_copy, const int64_t *sizes,
                                     int64_t ntensors, const float *param_norms,
                                     const float *update_norms, const float *lr,
                                     float weight_decay, int use_nvlamb, const int *noop_flag,
                                     int dtype_update, int dtype_param, void *stream);

/* ---- test hook of the dropout mask definition (no counterpart in the
 * reference; tests/ compare it with the integer Philox oracle) ------------- */

/* Writes the keep mask (1 = kept) of n elements as uint8. */
int oslo_philox_mask(uint8_t *mask_out, int64_t n, float p, uint64_t seed,
                     uint64_t offset, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* OSLO_HIP_H */
