// C-ABI entry points of the scaled causal, padding-masked and additive-term
// softmax, forward and backward (kernels and launchers: softmax_kernels.hip.h,
// instantiated by softmax_inst.hip).
//
// Entry-point shapes follow
// oslo/torch/_C/csrc/FusedScaleMaskSoftmaxBinder.cpp:39-105.
#include "softmax_kernels.hip.h"

namespace oslo {

OSLO_SM_FWD_INSTANCES(extern, float)
OSLO_SM_FWD_INSTANCES(extern, _Float16)
OSLO_SM_FWD_INSTANCES(extern, __bf16)
OSLO_SM_BWD_INSTANCES(extern, float)
OSLO_SM_BWD_INSTANCES(extern, _Float16)
OSLO_SM_BWD_INSTANCES(extern, __bf16)

#define OSLO_SM_DISPATCH(dtype, MODE, FN, ...)                       \
  do {                                                               \
    if (dtype == OSLO_DTYPE_F32) return FN<float, MODE>(__VA_ARGS__); \
    if (dtype == OSLO_DTYPE_F16) return FN<_Float16, MODE>(__VA_ARGS__); \
    return FN<__bf16, MODE>(__VA_ARGS__);                            \
  } while (0)

static int check_softmax_shape(const char *what, int64_t rows_outer, int64_t sq,
                               int64_t sk, int dtype) {
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: unknown dtype %d", what, dtype);
  if (rows_outer < 0 || sq < 0 || sk < 1 || sq > 0x7fffffff || sk > 0x7fffffff)
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: bad shape [%lld, %lld, %lld]",
                what, (long long)rows_outer, (long long)sq, (long long)sk);
  return OSLO_OK;
}

static int check_dropout_p(const char *what, float p) {
  if (!(p >= 0.f && p <= 1.f))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: p = %g outside [0, 1]", what,
                (double)p);
  return OSLO_OK;
}

}  // namespace oslo

extern "C" {

using namespace oslo;

int oslo_softmax_causal_fwd(const void *x, void *y, int64_t attn_batches,
                            int64_t sq, int64_t sk, float scale, int dtype,
                            void *stream) {
  oslo::tune_snapshot();
  int rc = check_softmax_shape("softmax causal fwd", attn_batches, sq, sk, dtype);
  if (rc != OSLO_OK) return rc;
  if (attn_batches * sq == 0) return OSLO_OK;
  OSLO_REQUIRE(x && y, "softmax causal fwd: null tensor pointer");
  SoftmaxGeom g{attn_batches * sq, (int)sq, (int)sk, 1, 0, 0, 1, 1};
  OSLO_SM_DISPATCH(dtype, kModeCausal, launch_softmax_fwd, x, nullptr, y,
                   nullptr, DropArgs{}, g, scale, (hipStream_t)stream);
}

int oslo_softmax_causal_bwd(const void *dy, const void *y, void *dx,
                            int64_t attn_batches, int64_t sq, int64_t sk,
                            float scale, int dtype, void *stream) {
  oslo::tune_snapshot();
  int rc = check_softmax_shape("softmax causal bwd", attn_batches, sq, sk, dtype);
  if (rc != OSLO_OK) return rc;
  if (attn_batches * sq == 0) return OSLO_OK;
  OSLO_REQUIRE(dy && y && dx, "softmax causal bwd: null tensor pointer");
  SoftmaxGeom g{attn_batches * sq, (int)sq, (int)sk, 1, 0, 0, 1, 1};
  OSLO_SM_DISPATCH(dtype, kModeCausal, launch_softmax_bwd, dy, y, nullptr, dx,
                   g, scale, (hipStream_t)stream);
}

static int masked_geom(const char *what, int64_t b, int64_t np, int64_t sq,
                       int64_t sk, int64_t mask_b, int64_t mask_sq,
                       SoftmaxGeom *g, int causal = 0) {
  if (b < 0 || np < 0 || np > 0x7fffffff)
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: bad batch/head count", what);
  if (!(mask_b == 1 || mask_b == b) || !(mask_sq == 1 || mask_sq == sq))
    return fail(OSLO_ERR_INVALID_ARGUMENT,
                "%s: mask shape [%lld,1,%lld,%lld] does not broadcast to "
                "[%lld,%lld,%lld,%lld]",
                what, (long long)mask_b, (long long)mask_sq, (long long)sk,
                (long long)b, (long long)np, (long long)sq, (long long)sk);
  *g = SoftmaxGeom{b * np * sq,
                   (int)sq,
                   (int)sk,
                   (int)(np > 0 ? np : 1),
                   (int)(mask_b == 1 ? 0 : mask_sq),
                   (int)(mask_sq == sq && sq != 1 ? 1 : 0),
                   1,
                   1,
                   causal};
  return OSLO_OK;
}

static int masked_fwd_entry(const char *what, int causal, const void *x,
                            const uint8_t *mask, void *y, int64_t b, int64_t np,
                            int64_t sq, int64_t sk, int64_t mask_b,
                            int64_t mask_sq, float scale, int dtype,
                            void *stream) {
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc != OSLO_OK) return rc;
  SoftmaxGeom g;
  rc = masked_geom(what, b, np, sq, sk, mask_b, mask_sq, &g, causal);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(x && y && mask, "%s: null tensor pointer", what);
  OSLO_SM_DISPATCH(dtype, kModeMasked, launch_softmax_fwd, x, mask, y, nullptr,
                   DropArgs{}, g, scale, (hipStream_t)stream);
}

static int masked_bwd_entry(const char *what, int causal, const void *dy,
                            const void *y, const uint8_t *mask, void *dx,
                            int64_t b, int64_t np, int64_t sq, int64_t sk,
                            int64_t mask_b, int64_t mask_sq, float scale,
                            int dtype, void *stream) {
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc != OSLO_OK) return rc;
  SoftmaxGeom g;
  if (mask == nullptr) {
    mask_b = 1;
    mask_sq = 1;
  }
  rc = masked_geom(what, b, np, sq, sk, mask_b, mask_sq, &g, causal);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(dy && y && dx, "%s: null tensor pointer", what);
  // without the mask every key is read: a row that had no visible key holds
  // the uniform distribution, beyond the diagonal too
  if (mask == nullptr)
    OSLO_SM_DISPATCH(dtype, kModeDense, launch_softmax_bwd, dy, y, nullptr, dx,
                     g, scale, (hipStream_t)stream);
  OSLO_SM_DISPATCH(dtype, kModeMasked, launch_softmax_bwd, dy, y, mask, dx, g,
                   scale, (hipStream_t)stream);
}

int oslo_softmax_masked_fwd(const void *x, const uint8_t *mask, void *y,
                            int64_t b, int64_t np, int64_t sq, int64_t sk,
                            int64_t mask_b, int64_t mask_sq, float scale,
                            int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_fwd_entry("softmax masked fwd", 0, x, mask, y, b, np, sq, sk,
                          mask_b, mask_sq, scale, dtype, stream);
}

int oslo_softmax_masked_bwd(const void *dy, const void *y, const uint8_t *mask,
                            void *dx, int64_t b, int64_t np, int64_t sq,
                            int64_t sk, int64_t mask_b, int64_t mask_sq,
                            float scale, int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_bwd_entry("softmax masked bwd", 0, dy, y, mask, dx, b, np, sq,
                          sk, mask_b, mask_sq, scale, dtype, stream);
}

int oslo_softmax_causal_masked_fwd(const void *x, const uint8_t *mask, void *y,
                                   int64_t b, int64_t np, int64_t sq,
                                   int64_t sk, int64_t mask_b, int64_t mask_sq,
                                   float scale, int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_fwd_entry("softmax causal masked fwd", 1, x, mask, y, b, np, sq,
                          sk, mask_b, mask_sq, scale, dtype, stream);
}

int oslo_softmax_causal_masked_bwd(const void *dy, const void *y,
                                   const uint8_t *mask, void *dx, int64_t b,
                                   int64_t np, int64_t sq, int64_t sk,
                                   int64_t mask_b, int64_t mask_sq, float scale,
                                   int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_bwd_entry("softmax causal masked bwd", 1, dy, y, mask, dx, b,
                          np, sq, sk, mask_b, mask_sq, scale, dtype, stream);
}

// ---- additive floating-point term ------------------------------------------
static int bias_geom(const char *what, int64_t b, int64_t np, int64_t sq,
                     int64_t sk, const void *bias, int64_t sb, int64_t sh,
                     int64_t sq_stride, int bias_dtype, int flags, int dtype,
                     SoftmaxGeom *g) {
  if (b < 0 || np < 0 || np > 0x7fffffff)
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: bad batch/head count", what);
  if ((flags & ~(OSLO_SOFTMAX_CAUSAL | OSLO_SOFTMAX_SKIP_HIDDEN)) != 0)
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: unknown flag bits 0x%x", what, flags);
  if (bias != nullptr) {
    if (bias_dtype != dtype && bias_dtype != OSLO_DTYPE_F32)
      return fail(OSLO_ERR_INVALID_ARGUMENT,
                  "%s: the additive term must have the logits' dtype or float32", what);
    if (sb < 0 || sh < 0 || sq_stride < 0)
      return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: negative stride of the additive term", what);
  }
  *g = SoftmaxGeom{b * np * sq, (int)sq, (int)sk, (int)(np > 0 ? np : 1), 0, 0, 1, 1,
                   (flags & OSLO_SOFTMAX_CAUSAL) ? 1 : 0};
  g->bias_sb = sb;
  g->bias_sh = sh;
  g->bias_sq = sq_stride;
  g->bias_esize = dtype_size(bias_dtype);
  g->bias_skip = (flags & OSLO_SOFTMAX_SKIP_HIDDEN) ? 1 : 0;
  // a term with a row per head or query that the whole batch shares (a
  // position bias): the batch entries of one row of it run next to each other
  if (bias != nullptr && sb == 0 && b > 1 && b <= 0x7fffffff && (sh != 0 || sq_stride != 0) &&
      g_tune.softmax_bias_order != 1) {
    g->batch_inner = 1;
    g->nb = (int)b;
    g->hq_rows = np * sq;
    // (runs of 2^group_shift consecutive rows of one batch entry, then the same
    //  rows of the next entry)
    int group = g_tune.softmax_bias_group > 0 ? g_tune.softmax_bias_group : 32;
    while (group > 1 && g->hq_rows % group != 0) group >>= 1;
    while ((1 << g->group_shift) < group) ++g->group_shift;
  }
  return OSLO_OK;
}

int oslo_softmax_bias_fwd(const void *x, const void *bias, void *y, int64_t b,
                          int64_t np, int64_t sq, int64_t sk,
                          int64_t bias_stride_b, int64_t bias_stride_h,
                          int64_t bias_stride_q, int bias_dtype, int flags,
                          float scale, int dtype, void *stream) {
  oslo::tune_snapshot();
  const char *what = "softmax bias fwd";
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(b * np * sq == 0 || bias, "%s: null additive term", what);
  SoftmaxGeom g;
  rc = bias_geom(what, b, np, sq, sk, bias, bias_stride_b, bias_stride_h,
                 bias_stride_q, bias_dtype, flags, dtype, &g);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(x && y, "%s: null tensor pointer", what);
  OSLO_SM_DISPATCH(dtype, kModeBias, launch_softmax_fwd, x, (const uint8_t *)bias,
                   y, nullptr, DropArgs{}, g, scale, (hipStream_t)stream);
}

int oslo_softmax_bias_bwd(const void *dy, const void *y, const void *bias,
                          void *dx, int64_t b, int64_t np, int64_t sq,
                          int64_t sk, int64_t bias_stride_b,
                          int64_t bias_stride_h, int64_t bias_stride_q,
                          int bias_dtype, int flags, float scale, int dtype,
                          void *stream) {
  oslo::tune_snapshot();
  const char *what = "softmax bias bwd";
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc != OSLO_OK) return rc;
  SoftmaxGeom g;
  rc = bias_geom(what, b, np, sq, sk, bias, bias_stride_b, bias_stride_h,
                 bias_stride_q, bias != nullptr ? bias_dtype : dtype, flags, dtype, &g);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(dy && y && dx, "%s: null tensor pointer", what);
  // the term only serves to skip loads: without it (or without the flag) the
  // rows are read up to the diagonal, or in full
  if (bias == nullptr || !g.bias_skip) {
    if (g.causal) {
      SoftmaxGeom c{g.rows, (int)sq, (int)sk, 1, 0, 0, 1, 1};
      OSLO_SM_DISPATCH(dtype, kModeCausal, launch_softmax_bwd, dy, y, nullptr,
                       dx, c, scale, (hipStream_t)stream);
    }
    OSLO_SM_DISPATCH(dtype, kModeDense, launch_softmax_bwd, dy, y, nullptr, dx,
                     g, scale, (hipStream_t)stream);
  }
  OSLO_SM_DISPATCH(dtype, kModeBias, launch_softmax_bwd, dy, y,
                   (const uint8_t *)bias, dx, g, scale, (hipStream_t)stream);
}

int oslo_softmax_bias_dropout_fwd(const void *x, const void *bias, void *out,
                                  float *stats, int64_t b, int64_t np,
                                  int64_t sq, int64_t sk, int64_t bias_stride_b,
                                  int64_t bias_stride_h, int64_t bias_stride_q,
                                  int bias_dtype, int flags, float scale,
                                  float p, uint64_t seed, uint64_t offset,
                                  int dtype, void *stream) {
  oslo::tune_snapshot();
  const char *what = "softmax bias dropout fwd";
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc == OSLO_OK) rc = check_dropout_p(what, p);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(b * np * sq == 0 || bias, "%s: null additive term", what);
  SoftmaxGeom g;
  rc = bias_geom(what, b, np, sq, sk, bias, bias_stride_b, bias_stride_h,
                 bias_stride_q, bias_dtype, flags, dtype, &g);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(x && out && stats, "%s: null pointer", what);
  OSLO_SM_DISPATCH(dtype, kModeBias, launch_softmax_fwd, x, (const uint8_t *)bias,
                   out, stats, make_drop(p, seed, offset), g, scale,
                   (hipStream_t)stream);
}

int oslo_softmax_bias_dropout_bwd(const void *dout, const void *x,
                                  const void *bias, const float *stats,
                                  void *dx, int64_t b, int64_t np, int64_t sq,
                                  int64_t sk, int64_t bias_stride_b,
                                  int64_t bias_stride_h, int64_t bias_stride_q,
                                  int bias_dtype, int flags, float scale,
                                  float p, uint64_t seed, uint64_t offset,
                                  int dtype, void *stream) {
  oslo::tune_snapshot();
  const char *what = "softmax bias dropout bwd";
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc == OSLO_OK) rc = check_dropout_p(what, p);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(b * np * sq == 0 || bias, "%s: null additive term", what);
  SoftmaxGeom g;
  rc = bias_geom(what, b, np, sq, sk, bias, bias_stride_b, bias_stride_h,
                 bias_stride_q, bias_dtype, flags, dtype, &g);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(dout && x && stats && dx, "%s: null pointer", what);
  OSLO_SM_DISPATCH(dtype, kModeBias, launch_softmax_dropout_bwd, dout, x, stats,
                   (const uint8_t *)bias, dx, make_drop(p, seed, offset), g,
                   scale, (hipStream_t)stream);
}

int oslo_softmax_batch_per_block(int64_t sq, int64_t sk, int64_t b,
                                 int64_t np) {
  oslo::tune_snapshot();
  if (sq < 1 || sk < 1 || b < 1 || np < 1)
    return fail(OSLO_ERR_INVALID_ARGUMENT,
                "softmax_batch_per_block: bad shape");
  // rows per workgroup of the 16-bit masked kernel (the reference's shim only
  // admits fp16 / bf16); rows that do not vectorise run one row per workgroup
  SoftmaxPlan pl = plan_softmax(sk, 8, 32, 2, 4);
  if (!pl.ok) pl = plan_softmax(sk, 8, kFwdMaxElems, 2, 4);
  if (!pl.ok) return 1;
  return pl.rpb * pl.rpw * (kWave / pl.lpr);
}


int oslo_softmax_causal_dropout_fwd(const void *x, void *out, float *stats,
                                    int64_t attn_batches, int64_t sq,
                                    int64_t sk, float scale, float p,
                                    uint64_t seed, uint64_t offset, int dtype,
                                    void *stream) {
  oslo::tune_snapshot();
  const char *what = "softmax causal dropout fwd";
  int rc = check_softmax_shape(what, attn_batches, sq, sk, dtype);
  if (rc == OSLO_OK) rc = check_dropout_p(what, p);
  if (rc != OSLO_OK) return rc;
  if (attn_batches * sq == 0) return OSLO_OK;
  OSLO_REQUIRE(x && out && stats, "softmax causal dropout fwd: null pointer");
  SoftmaxGeom g{attn_batches * sq, (int)sq, (int)sk, 1, 0, 0, 1, 1};
  OSLO_SM_DISPATCH(dtype, kModeCausal, launch_softmax_fwd, x, nullptr, out,
                   stats, make_drop(p, seed, offset), g, scale,
                   (hipStream_t)stream);
}

int oslo_softmax_causal_dropout_bwd(const void *dout, const void *x,
                                    const float *stats, void *dx,
                                    int64_t attn_batches, int64_t sq,
                                    int64_t sk, float scale, float p,
                                    uint64_t seed, uint64_t offset, int dtype,
                                    void *stream) {
  oslo::tune_snapshot();
  const char *what = "softmax causal dropout bwd";
  int rc = check_softmax_shape(what, attn_batches, sq, sk, dtype);
  if (rc == OSLO_OK) rc = check_dropout_p(what, p);
  if (rc != OSLO_OK) return rc;
  if (attn_batches * sq == 0) return OSLO_OK;
  OSLO_REQUIRE(dout && x && stats && dx,
               "softmax causal dropout bwd: null pointer");
  SoftmaxGeom g{attn_batches * sq, (int)sq, (int)sk, 1, 0, 0, 1, 1};
  OSLO_SM_DISPATCH(dtype, kModeCausal, launch_softmax_dropout_bwd, dout, x,
                   stats, nullptr, dx, make_drop(p, seed, offset), g, scale,
                   (hipStream_t)stream);
}

static int masked_dropout_fwd_entry(const char *what, int causal, const void *x,
                                    const uint8_t *mask, void *out, float *stats,
                                    int64_t b, int64_t np, int64_t sq,
                                    int64_t sk, int64_t mask_b, int64_t mask_sq,
                                    float scale, float p, uint64_t seed,
                                    uint64_t offset, int dtype, void *stream) {
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc == OSLO_OK) rc = check_dropout_p(what, p);
  if (rc != OSLO_OK) return rc;
  SoftmaxGeom g;
  rc = masked_geom(what, b, np, sq, sk, mask_b, mask_sq, &g, causal);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(x && out && mask && stats, "%s: null pointer", what);
  OSLO_SM_DISPATCH(dtype, kModeMasked, launch_softmax_fwd, x, mask, out, stats,
                   make_drop(p, seed, offset), g, scale, (hipStream_t)stream);
}

static int masked_dropout_bwd_entry(const char *what, int causal,
                                    const void *dout, const void *x,
                                    const uint8_t *mask, const float *stats,
                                    void *dx, int64_t b, int64_t np, int64_t sq,
                                    int64_t sk, int64_t mask_b, int64_t mask_sq,
                                    float scale, float p, uint64_t seed,
                                    uint64_t offset, int dtype, void *stream) {
  int rc = check_softmax_shape(what, b, sq, sk, dtype);
  if (rc == OSLO_OK) rc = check_dropout_p(what, p);
  if (rc != OSLO_OK) return rc;
  SoftmaxGeom g;
  rc = masked_geom(what, b, np, sq, sk, mask_b, mask_sq, &g, causal);
  if (rc != OSLO_OK) return rc;
  if (g.rows == 0) return OSLO_OK;
  OSLO_REQUIRE(dout && x && mask && stats && dx, "%s: null pointer", what);
  OSLO_SM_DISPATCH(dtype, kModeMasked, launch_softmax_dropout_bwd, dout, x,
                   stats, mask, dx, make_drop(p, seed, offset), g, scale,
                   (hipStream_t)stream);
}

int oslo_softmax_masked_dropout_fwd(const void *x, const uint8_t *mask,
                                    void *out, float *stats, int64_t b,
                                    int64_t np, int64_t sq, int64_t sk,
                                    int64_t mask_b, int64_t mask_sq,
                                    float scale, float p, uint64_t seed,
                                    uint64_t offset, int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_dropout_fwd_entry("softmax masked dropout fwd", 0, x, mask, out,
                                  stats, b, np, sq, sk, mask_b, mask_sq, scale,
                                  p, seed, offset, dtype, stream);
}

int oslo_softmax_masked_dropout_bwd(const void *dout, const void *x,
                                    const uint8_t *mask, const float *stats,
                                    void *dx, int64_t b, int64_t np, int64_t sq,
                                    int64_t sk, int64_t mask_b, int64_t mask_sq,
                                    float scale, float p, uint64_t seed,
                                    uint64_t offset, int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_dropout_bwd_entry("softmax masked dropout bwd", 0, dout, x,
                                  mask, stats, dx, b, np, sq, sk, mask_b,
                                  mask_sq, scale, p, seed, offset, dtype,
                                  stream);
}

int oslo_softmax_causal_masked_dropout_fwd(const void *x, const uint8_t *mask,
                                           void *out, float *stats, int64_t b,
                                           int64_t np, int64_t sq, int64_t sk,
                                           int64_t mask_b, int64_t mask_sq,
                                           float scale, float p, uint64_t seed,
                                           uint64_t offset, int dtype,
                                           void *stream) {
  oslo::tune_snapshot();
  return masked_dropout_fwd_entry("softmax causal masked dropout fwd", 1, x,
                                  mask, out, stats, b, np, sq, sk, mask_b,
                                  mask_sq, scale, p, seed, offset, dtype,
                                  stream);
}

int oslo_softmax_causal_masked_dropout_bwd(const void *dout, const void *x,
                                           const uint8_t *mask,
                                           const float *stats, void *dx,
                                           int64_t b, int64_t np, int64_t sq,
                                           int64_t sk, int64_t mask_b,
                                           int64_t mask_sq, float scale, float p,
                                           uint64_t seed, uint64_t offset,
                                           int dtype, void *stream) {
  oslo::tune_snapshot();
  return masked_dropout_bwd_entry("softmax causal masked dropout bwd", 1, dout,
                                  x, mask, stats, dx, b, np, sq, sk, mask_b,
                                  mask_sq, scale, p, seed, offset, dtype,
                                  stream);
}

}
