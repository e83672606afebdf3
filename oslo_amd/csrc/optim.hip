// Multi-tensor Adam / AdamW step for gfx950.
//
// One launch updates up to kMaxTensors parameter tensors: the tensor table
// (four pointers and a length per tensor, plus the prefix sums of the
// workgroups each tensor takes) travels in the kernel arguments, so nothing
// is staged in device memory.  A workgroup owns one short contiguous piece of
// one tensor -- a few 128-bit vectors per lane of each of g, p, m, v -- and
// exits: the launch is a plain streaming pass (28 bytes per fp32 element,
// 14 per 16-bit element).  Arithmetic follows
// oslo/torch/_C/csrc/multi_tensor_adam.cu:22-110 of the reference: fp32 math,
// mode 0 = L2 regularisation (the decay joins the gradient), mode 1 =
// decoupled weight decay (AdamW).
#include <math.h>

#include "capi.h"
#include "common.hip.h"

namespace oslo {

constexpr int kMaxTensors = 64;
constexpr int kAdamThreads = 256;

struct AdamTable {
  void *g[kMaxTensors];
  void *p[kMaxTensors];
  void *m[kMaxTensors];
  void *v[kMaxTensors];
  int64_t n[kMaxTensors];
  int64_t first_block[kMaxTensors + 1];  // prefix sums of workgroups
  int ntensors;
};

struct AdamArgs {
  float beta1, beta2, bc1, bc2, eps, lr, decay;
  int mode;
};

__device__ __forceinline__ void adam_update(float g, float &p, float &m,
                                            float &v, const AdamArgs &a) {
  // multi_tensor_adam.cu:78-96, term for term
  if (a.mode == 0) g = g + a.decay * p;
  m = a.beta1 * m + (1.f - a.beta1) * g;
  v = a.beta2 * v + (1.f - a.beta2) * g * g;
  const float mh = m / a.bc1;
  const float vh = v / a.bc2;
  const float denom = sqrtf(vh) + a.eps;
  float update = mh / denom;
  if (a.mode != 0) update = update + a.decay * p;
  p = p - a.lr * update;
}

template <typename T, int kAdamUnroll>
__global__ __launch_bounds__(kAdamThreads) void multi_tensor_adam_kernel(
    AdamTable tab, AdamArgs a) {
  constexpr int E = io<T>::EPV;
  constexpr int64_t kPiece = (int64_t)kAdamThreads * kAdamUnroll * E;
  // which tensor does this workgroup belong to (uniform: scalar search)
  const int64_t b = blockIdx.x;
  int t = 0;
  while (t + 1 < tab.ntensors && tab.first_block[t + 1] <= b) ++t;
  const int64_t piece = b - tab.first_block[t];
  const int64_t n = tab.n[t];
  const int64_t start = piece * kPiece;
  const T *g = static_cast<const T *>(tab.g[t]);
  T *p = static_cast<T *>(tab.p[t]);
  T *m = static_cast<T *>(tab.m[t]);
  T *v = static_cast<T *>(tab.v[t]);
  const bool aligned = ((reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(p) |
                         reinterpret_cast<uintptr_t>(m) | reinterpret_cast<uintptr_t>(v)) &
                        15u) == 0;
  if (aligned && start + kPiece <= n) {
    // full piece: kAdamUnroll vectors per lane and operand, all loads first
    float rg[kAdamUnroll][E], rp[kAdamUnroll][E], rm[kAdamUnroll][E], rv[kAdamUnroll][E];
#pragma unroll
    for (int u = 0; u < kAdamUnroll; ++u) {
      const int64_t i = start + ((int64_t)u * kAdamThreads + threadIdx.x) * E;
      load_chunk<T, E>(g + i, rg[u]);
      load_chunk<T, E>(p + i, rp[u]);
      load_chunk<T, E>(m + i, rm[u]);
      load_chunk<T, E>(v + i, rv[u]);
    }
#pragma unroll
    for (int u = 0; u < kAdamUnroll; ++u) {
      const int64_t i = start + ((int64_t)u * kAdamThreads + threadIdx.x) * E;
#pragma unroll
      for (int e = 0; e < E; ++e) adam_update(rg[u][e], rp[u][e], rm[u][e], rv[u][e], a);
      store_chunk<T, E>(p + i, rp[u]);
      store_chunk<T, E>(m + i, rm[u]);
      store_chunk<T, E>(v + i, rv[u]);
    }
    return;
  }
  // last piece of a tensor, or a tensor whose storage is not 16-byte aligned
  const int64_t end = start + kPiece < n ? start + kPiece : n;
  for (int64_t i = start + threadIdx.x; i < end; i += kAdamThreads) {
    const float gg = io<T>::from_scalar(g[i]);
    float pp = io<T>::from_scalar(p[i]);
    float mm = io<T>::from_scalar(m[i]);
    float vv = io<T>::from_scalar(v[i]);
    adam_update(gg, pp, mm, vv, a);
    p[i] = io<T>::to_scalar(pp);
    m[i] = io<T>::to_scalar(mm);
    v[i] = io<T>::to_scalar(vv);
  }
}

template <typename T, int kAdamUnroll>
static int launch_adam(const void *const *g, void *const *p, void *const *m,
                       void *const *v, const int64_t *sizes, int64_t ntensors,
                       const AdamArgs &a, hipStream_t st) {
  constexpr int64_t kPiece = (int64_t)kAdamThreads * kAdamUnroll * io<T>::EPV;
  AdamTable tab;
  tab.ntensors = 0;
  tab.first_block[0] = 0;
  auto flush = [&]() -> int {
    if (tab.ntensors == 0) return OSLO_OK;
    const int64_t blocks = tab.first_block[tab.ntensors];
    if (blocks > 0) {
      if (blocks > max_workgroups(kAdamThreads))
        return fail(OSLO_ERR_UNSUPPORTED, "multi_tensor_adam: a tensor too large for one launch");
      multi_tensor_adam_kernel<T, kAdamUnroll>
          <<<dim3((unsigned)blocks), kAdamThreads, 0, st>>>(tab, a);
      const int rc = check_launch("multi_tensor_adam_kernel");
      if (rc != OSLO_OK) return rc;
    }
    tab.ntensors = 0;
    return OSLO_OK;
  };
  for (int64_t i = 0; i < ntensors; ++i) {
    if (sizes[i] == 0) continue;
    if (sizes[i] < 0)
      return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_adam: tensor %lld has size %lld",
                  (long long)i, (long long)sizes[i]);
    if (!g[i] || !p[i] || !m[i] || !v[i])
      return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_adam: tensor %lld has a null pointer",
                  (long long)i);
    // one launch stays below 2^32 work-items
    if (tab.ntensors > 0 &&
        tab.first_block[tab.ntensors] + ceil_div(sizes[i], kPiece) > max_workgroups(kAdamThreads)) {
      const int rc = flush();
      if (rc != OSLO_OK) return rc;
    }
    const int k = tab.ntensors;
    tab.g[k] = const_cast<void *>(g[i]);
    tab.p[k] = p[i];
    tab.m[k] = m[i];
    tab.v[k] = v[i];
    tab.n[k] = sizes[i];
    tab.first_block[k + 1] = tab.first_block[k] + ceil_div(sizes[i], kPiece);
    tab.ntensors = k + 1;
    if (tab.ntensors == kMaxTensors) {
      const int rc = flush();
      if (rc != OSLO_OK) return rc;
    }
  }
  return flush();
}

}  // namespace oslo

extern "C" {

int oslo_multi_tensor_adam(const void *const *g, void *const *p, void *const *m,
                           void *const *v, const int64_t *sizes,
                           int64_t ntensors, float lr, float beta1, float beta2,
                           float eps, int step, int mode, int bias_correction,
                           float weight_decay, int dtype, void *stream) {
  oslo::tune_snapshot();
  using namespace oslo;
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_adam: unknown dtype %d", dtype);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_adam: negative tensor count");
  OSLO_REQUIRE(mode == 0 || mode == 1, "multi_tensor_adam: mode %d is neither 0 (L2) nor 1 (AdamW)",
               mode);
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(g && p && m && v && sizes, "multi_tensor_adam: null table pointer");
  AdamArgs a;
  a.beta1 = beta1;
  a.beta2 = beta2;
  a.eps = eps;
  a.lr = lr;
  a.decay = weight_decay;
  a.mode = mode;
  // multi_tensor_adam.cu:120-125: 1 - beta^step, evaluated by std::pow on the
  // float betas (which promotes to double) and stored as float
  a.bc1 = 1.0f;
  a.bc2 = 1.0f;
  if (bias_correction == 1) {
    a.bc1 = (float)(1.0 - pow((double)beta1, (double)step));
    a.bc2 = (float)(1.0 - pow((double)beta2, (double)step));
  }
  hipStream_t st = (hipStream_t)stream;
  // 128-bit vectors per lane and operand: 1, 2 and 4 measure within 2 % of
  // each other on MI355X (5.6-5.8 TB/s)
  const int unroll = g_tune.adam_unroll == 1 || g_tune.adam_unroll == 2 || g_tune.adam_unroll == 4
                         ? g_tune.adam_unroll
                         : 4;
#define OSLO_ADAM(T_)                                                           \
  (unroll == 1   ? launch_adam<T_, 1>(g, p, m, v, sizes, ntensors, a, st)       \
   : unroll == 2 ? launch_adam<T_, 2>(g, p, m, v, sizes, ntensors, a, st)       \
                 : launch_adam<T_, 4>(g, p, m, v, sizes, ntensors, a, st))
  if (dtype == OSLO_DTYPE_F32) return OSLO_ADAM(float);
  if (dtype == OSLO_DTYPE_F16) return OSLO_ADAM(_Float16);
  return OSLO_ADAM(__bf16);
#undef OSLO_ADAM
}

}  // extern "C"
