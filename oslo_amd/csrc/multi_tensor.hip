// Multi-tensor optimizer steps and norms for gfx950: SGD, Adagrad, NovoGrad,
// the two stages of LAMB and the L2 / max norms they need.
//
// The launch scheme is that of the Adam step (optim.hip): the tensor table of a
// launch -- one pointer per operand list and a length per tensor, plus the
// prefix sums of the workgroups each tensor takes -- travels in the kernel
// arguments, a workgroup owns one short contiguous piece of one tensor, loads
// a few 128-bit vectors per lane of every operand, updates them in fp32 and
// exits.  Every launch is a plain streaming pass.  The arithmetic of each
// update follows the reference's functor term for term (cited at each one).
#include <math.h>

#include <tuple>

#include "capi.h"
#include "common.hip.h"

namespace oslo {

constexpr int kMtThreads = 256;
constexpr int kMtMaxTensors = 48;
constexpr int kMtUnroll = 4;

template <int NL> struct MtTable {
  void *a[NL][kMtMaxTensors];
  int64_t n[kMtMaxTensors];
  int64_t first_block[kMtMaxTensors + 1];  // prefix sums of workgroups
  int tidx[kMtMaxTensors];                 // index of the tensor in the caller's lists
  int64_t block0;                          // workgroups of the launches before this one
  int ntensors;
};

// Tensor of workgroup b (uniform: a scalar search).  Tensors without elements
// take no workgroup and are stepped over.
template <int NL>
__device__ __forceinline__ int mt_find_tensor(const MtTable<NL> &tab, int64_t b) {
  int t = 0;
  while (t + 1 < tab.ntensors && tab.first_block[t + 1] <= b) ++t;
  return t;
}

// ---------------------------------------------------------------------------
// element-wise updates
// ---------------------------------------------------------------------------
// An update F names its operand lists (Types), how many elements a lane moves
// per vector step (E: one 128-bit vector of the narrowest type), which lists
// it reads and writes, an optional per-tensor context and the update of one
// element in fp32.
template <typename F, int L = 0>
__device__ __forceinline__ void mt_load(const F &f, void *const *base, int64_t i,
                                        float (&r)[F::NL][F::E]) {
  if constexpr (L < F::NL) {
    using T = std::tuple_element_t<L, typename F::Types>;
    if (f.reads(L)) {
      load_chunk<T, F::E>(static_cast<const T *>(base[L]) + i, r[L]);
    } else {
#pragma unroll
      for (int e = 0; e < F::E; ++e) r[L][e] = 0.f;
    }
    mt_load<F, L + 1>(f, base, i, r);
  }
}

template <typename F, int L = 0>
__device__ __forceinline__ void mt_store(const F &f, void *const *base, int64_t i,
                                         float (&r)[F::NL][F::E]) {
  if constexpr (L < F::NL) {
    using T = std::tuple_element_t<L, typename F::Types>;
    if (f.writes(L)) store_chunk<T, F::E>(static_cast<T *>(base[L]) + i, r[L]);
    mt_store<F, L + 1>(f, base, i, r);
  }
}

template <typename F, int L = 0>
__device__ __forceinline__ void mt_load1(const F &f, void *const *base, int64_t i,
                                         float (&v)[F::NL]) {
  if constexpr (L < F::NL) {
    using T = std::tuple_element_t<L, typename F::Types>;
    v[L] = f.reads(L) ? io<T>::from_scalar(static_cast<const T *>(base[L])[i]) : 0.f;
    mt_load1<F, L + 1>(f, base, i, v);
  }
}

template <typename F, int L = 0>
__device__ __forceinline__ void mt_store1(const F &f, void *const *base, int64_t i,
                                          float (&v)[F::NL]) {
  if constexpr (L < F::NL) {
    using T = std::tuple_element_t<L, typename F::Types>;
    if (f.writes(L)) static_cast<T *>(base[L])[i] = io<T>::to_scalar(v[L]);
    mt_store1<F, L + 1>(f, base, i, v);
  }
}

template <typename F>
__global__ __launch_bounds__(kMtThreads) void multi_tensor_apply_kernel(MtTable<F::NL> tab, F f) {
  constexpr int NL = F::NL, E = F::E, U = kMtUnroll;
  constexpr int64_t kPiece = (int64_t)kMtThreads * U * E;
  if (f.skip()) return;
  const int64_t b = blockIdx.x;
  const int t = mt_find_tensor(tab, b);
  const int64_t n = tab.n[t];
  const int64_t start = (b - tab.first_block[t]) * kPiece;
  const typename F::Ctx ctx = f.context(tab.tidx[t]);
  void *base[NL];
  uintptr_t bits = 0;
#pragma unroll
  for (int l = 0; l < NL; ++l) {
    base[l] = tab.a[l][t];
    bits |= reinterpret_cast<uintptr_t>(base[l]);
  }
  if ((bits & 15u) == 0 && start + kPiece <= n) {
    // full piece: U vectors per lane and operand, all loads first
    float r[U][NL][E];
#pragma unroll
    for (int u = 0; u < U; ++u)
      mt_load<F>(f, base, start + ((int64_t)u * kMtThreads + threadIdx.x) * E, r[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < E; ++e) {
        float v[NL];
#pragma unroll
        for (int l = 0; l < NL; ++l) v[l] = r[u][l][e];
        f.update(v, ctx);
#pragma unroll
        for (int l = 0; l < NL; ++l) r[u][l][e] = v[l];
      }
      mt_store<F>(f, base, start + ((int64_t)u * kMtThreads + threadIdx.x) * E, r[u]);
    }
    return;
  }
  // last piece of a tensor, or a tensor whose storage is not 16-byte aligned
  const int64_t end = start + kPiece < n ? start + kPiece : n;
  for (int64_t i = start + threadIdx.x; i < end; i += kMtThreads) {
    float v[NL];
    mt_load1<F>(f, base, i, v);
    f.update(v, ctx);
    mt_store1<F>(f, base, i, v);
  }
}

struct NoCtx {};

// base^exponent for a step count, by repeated squaring
__device__ __forceinline__ double int_power(double base, int exponent) {
  double r = 1.0;
  for (int e = exponent > 0 ? exponent : 0; e > 0; e >>= 1) {
    if (e & 1) r *= base;
    base *= base;
  }
  return r;
}

// SGD with momentum (oslo/torch/_C/csrc/multi_tensor_sgd.cu:29-122): lists
// gradient, weight, momentum buffer and, with OUT, a 16-bit copy of the
// updated weight.  The launch does nothing when *noop is non-zero (:35-36).
template <typename TG, typename TW, typename TO, bool OUT> struct SgdOp {
  static constexpr int NL = OUT ? 4 : 3;
  static constexpr int E = (sizeof(TG) == 2 || sizeof(TW) == 2 || OUT) ? 8 : 4;
  using Types = std::tuple<TG, TW, TW, TO>;
  using Ctx = NoCtx;
  float wd, momentum, dampening, lr, scale;
  int nesterov, first_run, wd_after_momentum;
  const int *noop;
  __device__ bool skip() const { return noop != nullptr && *noop != 0; }
  __device__ Ctx context(int) const { return Ctx(); }
  __device__ bool reads(int l) const { return l == 0 || l == 1 || (l == 2 && momentum != 0.f && !first_run); }
  __device__ bool writes(int l) const { return l == 1 || (l == 2 && momentum != 0.f) || l == 3; }
  __device__ void update(float (&v)[NL], const Ctx &) const {
    float g = v[0] * scale;
    const float w = v[1];
    float mom = v[2];
    if (wd != 0.f && !wd_after_momentum) g += wd * w;
    if (momentum != 0.f) {
      mom = first_run ? g : mom * momentum + (1.f - dampening) * g;
      g = nesterov ? g + momentum * mom : mom;
    }
    if (wd != 0.f && wd_after_momentum) g += wd * w;
    // the weight is rounded to its storage type first; the 16-bit copy is a
    // conversion of the stored weight (:108-113)
    v[1] = io<TW>::round(w + (-lr * g));
    v[2] = mom;
    if constexpr (OUT) v[3] = v[1] = pinned(v[1]);
  }
};

// Adagrad (oslo/torch/_C/csrc/multi_tensor_adagrad.cu:24-84): gradient,
// parameter, sum of squared gradients.
template <typename T> struct AdagradOp {
  static constexpr int NL = 3;
  static constexpr int E = io<T>::EPV;
  using Types = std::tuple<T, T, T>;
  using Ctx = NoCtx;
  float eps, lr, decay;
  int mode;
  __device__ bool skip() const { return false; }
  __device__ Ctx context(int) const { return Ctx(); }
  __device__ bool reads(int) const { return true; }
  __device__ bool writes(int l) const { return l != 0; }
  __device__ void update(float (&v)[NL], const Ctx &) const {
    float g = v[0], p = v[1], h = v[2];
    if (mode == 0) {  // L2
      g = g + decay * p;
      h = h + g * g;
      p = p - lr * (g / (sqrtf(h) + eps));
    } else {  // decoupled weight decay
      h = h + g * g;
      p = p - lr * (g / (sqrtf(h) + eps) + decay * p);
    }
    v[1] = p;
    v[2] = h;
  }
};

// NovoGrad (oslo/torch/_C/csrc/multi_tensor_novograd.cu:30-109): gradient,
// parameter, first moment; the second moment is one norm per tensor.
template <typename T> struct NovogradOp {
  static constexpr int NL = 3;
  static constexpr int E = io<T>::EPV;
  using Types = std::tuple<T, T, T>;
  struct Ctx {
    float denom;
  };
  float beta1, beta3, bc1, bc2, eps, lr, decay;
  int moment_mode;
  const float *grad_norms;
  __device__ bool skip() const { return false; }
  __device__ Ctx context(int tensor) const {
    Ctx c;
    c.denom = grad_norms[tensor] / bc2 + eps;
    return c;
  }
  __device__ bool reads(int) const { return true; }
  __device__ bool writes(int l) const { return l != 0; }
  __device__ void update(float (&v)[NL], const Ctx &c) const {
    float g = v[0], p = v[1], m = v[2];
    if (moment_mode == 0) {  // regularisation inside the moment
      g = (g / c.denom) + (decay * p);
      m = beta1 * m + beta3 * g;
      p = p - (lr * (m / bc1));
    } else {
      m = beta1 * m + beta3 * g;
      const float update = ((m / bc1) / c.denom) + (decay * p);
      p = p - (lr * update);
    }
    v[1] = p;
    v[2] = m;
  }
};

// LAMB, stage 1 (oslo/torch/_C/csrc/multi_tensor_lamb.cu:41-204): gradient,
// parameter, both moments; the update direction overwrites the gradient.
template <typename T> struct LambStage1Op {
  static constexpr int NL = 4;
  static constexpr int E = io<T>::EPV;
  using Types = std::tuple<T, T, T, T>;
  struct Ctx {
    float clip;
  };
  float beta1, beta2, beta3, bc1, bc2, eps, decay, max_global_grad_norm;
  int mode;
  const float *global_grad_norm;
  __device__ bool skip() const { return false; }
  __device__ Ctx context(int) const {
    Ctx c;
    const float gn = *global_grad_norm;
    c.clip = gn > max_global_grad_norm ? gn / max_global_grad_norm : 1.0f;
    return c;
  }
  __device__ bool reads(int l) const { return l != 1 || decay != 0.f; }
  __device__ bool writes(int l) const { return l != 1; }
  __device__ void update(float (&v)[NL], const Ctx &c) const {
    float g = v[0] / c.clip;
    const float p = v[1];
    float m = v[2], s = v[3];
    if (mode == 0) g = g + decay * p;  // L2 on the scaled gradient
    m = m * beta1 + beta3 * g;
    s = s * beta2 + (1.f - beta2) * g * g;
    float update = (m / bc1) / (sqrtf(s / bc2) + eps);
    if (mode != 0) update = update + (decay * p);
    v[0] = update;
    v[2] = m;
    v[3] = s;
  }
};

// LAMB, stage 2 (multi_tensor_lamb.cu:208-283): p -= ratio * update with the
// trust ratio of the tensor.
template <typename T> struct LambStage2Op {
  static constexpr int NL = 2;
  static constexpr int E = io<T>::EPV;
  using Types = std::tuple<T, T>;
  struct Ctx {
    float ratio;
  };
  float lr, decay;
  int use_nvlamb;
  const float *param_norms, *update_norms;
  __device__ bool skip() const { return false; }
  __device__ Ctx context(int tensor) const {
    Ctx c;
    c.ratio = lr;
    // the adaptive rate applies to every tensor with use_nvlamb, otherwise
    // only to those with weight decay
    if (use_nvlamb || decay != 0.f) {
      const float pn = param_norms[tensor], un = update_norms[tensor];
      c.ratio = (un != 0.f && pn != 0.f) ? lr * (pn / un) : lr;
    }
    return c;
  }
  __device__ bool reads(int) const { return true; }
  __device__ bool writes(int l) const { return l == 1; }
  __device__ void update(float (&v)[NL], const Ctx &c) const { v[1] = v[1] - (c.ratio * v[0]); }
};

// LAMB for mixed precision (oslo/torch/_C/csrc/multi_tensor_lamb_mp.cu): the
// step count, the learning rate, the clip threshold and the inverse loss scale
// live in device memory, so that a training step needs no host synchronisation,
// and both stages do nothing while the overflow flag is raised (:46-48, :246-248).
// Stage 1 (:40-205): gradients of type TG, parameter and moments of type TP
// (TG, or float32 master copies); the gradient is unscaled first.
template <typename TG, typename TP> struct LambMpStage1Op {
  static constexpr int NL = 4;
  static constexpr int E = (sizeof(TG) == 2 || sizeof(TP) == 2) ? 8 : 4;
  using Types = std::tuple<TG, TP, TP, TP>;
  struct Ctx {
    float clip, bc1, bc2, inv_scale;
  };
  float beta1, beta2, beta3, eps, decay;
  int mode, bias_correction;
  const int *step, *noop;
  const float *global_grad_norm, *max_global_grad_norm, *inv_scale;
  __device__ bool skip() const { return noop != nullptr && *noop != 0; }
  __device__ Ctx context(int) const {
    Ctx c;
    c.bc1 = 1.0f;
    c.bc2 = 1.0f;
    if (bias_correction == 1) {
      // in double, as the host forms them for the plain stages: 1 - beta^step
      // cancels, and a float32 power would leave 1 - 0.999^3 good to 2e-5 only
      const int s = *step;
      c.bc1 = (float)(1.0 - int_power((double)beta1, s));
      c.bc2 = (float)(1.0 - int_power((double)beta2, s));
    }
    const float gn = *global_grad_norm, mx = *max_global_grad_norm;
    c.clip = gn > mx ? gn / mx : 1.0f;
    c.inv_scale = *inv_scale;
    return c;
  }
  __device__ bool reads(int l) const { return l != 1 || decay != 0.f; }
  __device__ bool writes(int l) const { return l != 1; }
  __device__ void update(float (&v)[NL], const Ctx &c) const {
    float g = (v[0] * c.inv_scale) / c.clip;
    const float p = v[1];
    float m = v[2], s = v[3];
    if (mode == 0) g = g + decay * p;
    m = m * beta1 + beta3 * g;
    s = s * beta2 + (1.f - beta2) * g * g;
    float update = (m / c.bc1) / (sqrtf(s / c.bc2) + eps);
    if (mode != 0) update = update + (decay * p);
    v[0] = update;
    v[2] = m;
    v[3] = s;
  }
};

// Stage 2 (:209-328): update of type T, parameter of type TP and, with OUT, a
// copy of the new parameter in type T (the model's weights next to float32
// master weights).
template <typename T, typename TP, bool OUT> struct LambMpStage2Op {
  static constexpr int NL = OUT ? 3 : 2;
  static constexpr int E = (sizeof(T) == 2 || sizeof(TP) == 2) ? 8 : 4;
  using Types = std::tuple<T, TP, T>;
  struct Ctx {
    float ratio;
  };
  float decay;
  int use_nvlamb;
  const float *lr, *param_norms, *update_norms;
  const int *noop;
  __device__ bool skip() const { return noop != nullptr && *noop != 0; }
  __device__ Ctx context(int tensor) const {
    Ctx c;
    const float rate = *lr;
    c.ratio = rate;
    if (use_nvlamb || decay != 0.f) {
      const float pn = param_norms[tensor], un = update_norms[tensor];
      c.ratio = (un != 0.f && pn != 0.f) ? rate * (pn / un) : rate;
    }
    return c;
  }
  __device__ bool reads(int l) const { return l < 2; }
  __device__ bool writes(int l) const { return l >= 1; }
  __device__ void update(float (&v)[NL], const Ctx &c) const {
    v[1] = io<TP>::round(v[1] - (c.ratio * v[0]));
    if constexpr (OUT) v[2] = v[1] = pinned(v[1]);
  }
};

// ---------------------------------------------------------------------------
// norms (oslo/torch/_C/csrc/multi_tensor_l2norm.cu:29-98 L2, :102-172 max,
// clean-up kernels :174-255)
// ---------------------------------------------------------------------------
constexpr int kNormLoops = 4;

// Workgroup b reduces its piece to one value -- the sum of squares, or the
// largest magnitude with MAXNORM -- and stores it in partials[block0 + b].
// A value that is not finite raises *noop (every writer stores the same 1).
// With skip_if_flag the three norm kernels do nothing while *noop is raised
// (the "mp" variant, oslo/torch/_C/csrc/multi_tensor_l2norm_mp.cu:33-35, 113-115):
// the flag is read when a kernel starts, and every workgroup of the first
// kernel that finds it clear writes its partial value.
template <typename T, bool MAXNORM>
__global__ __launch_bounds__(kMtThreads) void multi_tensor_norm_kernel(MtTable<1> tab,
                                                                      float *__restrict__ partials,
                                                                      int *noop, int skip_if_flag) {
  constexpr int E = io<T>::EPV, U = kMtUnroll;
  if (skip_if_flag && *noop != 0) return;
  constexpr int64_t kStep = (int64_t)kMtThreads * U * E;
  constexpr int64_t kPiece = kStep * kNormLoops;
  __shared__ float red[kMtThreads / kWave];
  const int64_t b = blockIdx.x;
  const int t = mt_find_tensor(tab, b);
  const int64_t n = tab.n[t];
  const int64_t start = (b - tab.first_block[t]) * kPiece;
  const int64_t end = start + kPiece < n ? start + kPiece : n;
  const T *x = static_cast<const T *>(tab.a[0][t]);
  float acc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) acc[u] = 0.f;
  int64_t pos = start;
  if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    for (; pos + kStep <= end; pos += kStep) {
      float r[U][E];
#pragma unroll
      for (int u = 0; u < U; ++u)
        load_chunk<T, E>(x + pos + ((int64_t)u * kMtThreads + threadIdx.x) * E, r[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e)
          acc[u] = MAXNORM ? fmaxf(acc[u], fabsf(r[u][e])) : acc[u] + r[u][e] * r[u][e];
    }
  }
  for (int64_t i = pos + threadIdx.x; i < end; i += kMtThreads) {
    const float v = io<T>::from_scalar(x[i]);
    acc[0] = MAXNORM ? fmaxf(acc[0], fabsf(v)) : acc[0] + v * v;
  }
  float val = acc[0];
#pragma unroll
  for (int u = 1; u < U; ++u) val = MAXNORM ? fmaxf(val, acc[u]) : val + acc[u];
  val = MAXNORM ? wave_max(val) : wave_sum(val);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) red[wave] = val;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = red[0];
#pragma unroll
    for (int w = 1; w < kMtThreads / kWave; ++w) total = MAXNORM ? fmaxf(total, red[w]) : total + red[w];
    partials[tab.block0 + b] = total;
    if (noop != nullptr && !isfinite(total)) *noop = 1;
  }
}

// Workgroup t folds the partial values of tensor t in a fixed order and
// writes (blend == 0) or blends (blend == 1) the tensor's norm:
//   L2:  out = sqrt(sum)            or  sqrt(alpha * out^2 + beta * sum)
//   max: out = max                  or  alpha * out + beta * max
template <bool MAXNORM>
__global__ __launch_bounds__(kMtThreads) void multi_tensor_norm_finalize_kernel(
    MtTable<1> tab, const float *__restrict__ partials, float *__restrict__ out, int blend,
    float alpha, float beta, const int *noop, int skip_if_flag) {
  __shared__ float red[kMtThreads / kWave];
  if (skip_if_flag && *noop != 0) return;
  const int t = blockIdx.x;
  const int64_t lo = tab.block0 + tab.first_block[t], hi = tab.block0 + tab.first_block[t + 1];
  float val = 0.f;
  for (int64_t i = lo + threadIdx.x; i < hi; i += kMtThreads)
    val = MAXNORM ? fmaxf(val, partials[i]) : val + partials[i];
  val = MAXNORM ? wave_max(val) : wave_sum(val);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) red[wave] = val;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = red[0];
#pragma unroll
    for (int w = 1; w < kMtThreads / kWave; ++w) total = MAXNORM ? fmaxf(total, red[w]) : total + red[w];
    float *o = out + tab.tidx[t];
    if (MAXNORM)
      *o = blend ? alpha * (*o) + beta * total : total;
    else
      *o = blend ? sqrtf(alpha * (*o) * (*o) + beta * total) : sqrtf(total);
  }
}

// One workgroup folds all partial values into the norm over every tensor.
template <bool MAXNORM>
__global__ __launch_bounds__(1024) void multi_tensor_norm_global_kernel(
    const float *__restrict__ partials, int64_t total_blocks, float *__restrict__ out,
    const int *noop, int skip_if_flag) {
  __shared__ float red[1024 / kWave];
  if (skip_if_flag && *noop != 0) return;
  float val = 0.f;
  for (int64_t i = threadIdx.x; i < total_blocks; i += 1024)
    val = MAXNORM ? fmaxf(val, partials[i]) : val + partials[i];
  val = MAXNORM ? wave_max(val) : wave_sum(val);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) red[wave] = val;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = red[0];
    for (int w = 1; w < 1024 / kWave; ++w) total = MAXNORM ? fmaxf(total, red[w]) : total + red[w];
    *out = MAXNORM ? total : sqrtf(total);
  }
}

// ---------------------------------------------------------------------------
// host side: tables and launches
// ---------------------------------------------------------------------------
// Walks the tensors in order, fills tables of at most kMtMaxTensors tensors
// (and fewer than 2^32 work-items) and calls launch(table, workgroups) for each.
template <int NL, typename Launch>
static int mt_for_each_table(const char *what, void *const *const (&lists)[NL], const int64_t *sizes,
                             int64_t ntensors, int64_t piece, Launch &&launch) {
  MtTable<NL> tab;
  tab.ntensors = 0;
  tab.block0 = 0;
  tab.first_block[0] = 0;
  auto flush = [&]() -> int {
    if (tab.ntensors == 0) return OSLO_OK;
    const int64_t blocks = tab.first_block[tab.ntensors];
    const int rc = launch(tab, blocks);
    if (rc != OSLO_OK) return rc;
    tab.block0 += blocks;
    tab.ntensors = 0;
    return OSLO_OK;
  };
  for (int64_t i = 0; i < ntensors; ++i) {
    if (sizes[i] < 0)
      return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: tensor %lld has size %lld", what, (long long)i,
                  (long long)sizes[i]);
    const int64_t blocks = ceil_div(sizes[i], piece);
    if (blocks > max_workgroups(kMtThreads))
      return fail(OSLO_ERR_UNSUPPORTED, "%s: tensor %lld is too large for one launch", what, (long long)i);
    if (sizes[i] > 0)
      for (int l = 0; l < NL; ++l)
        if (lists[l][i] == nullptr)
          return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: tensor %lld of list %d is a null pointer", what,
                      (long long)i, l);
    if (tab.ntensors > 0 && tab.first_block[tab.ntensors] + blocks > max_workgroups(kMtThreads)) {
      const int rc = flush();
      if (rc != OSLO_OK) return rc;
    }
    const int k = tab.ntensors;
    for (int l = 0; l < NL; ++l) tab.a[l][k] = sizes[i] > 0 ? lists[l][i] : nullptr;
    tab.n[k] = sizes[i];
    tab.tidx[k] = (int)i;
    tab.first_block[k + 1] = tab.first_block[k] + blocks;
    tab.ntensors = k + 1;
    if (tab.ntensors == kMtMaxTensors) {
      const int rc = flush();
      if (rc != OSLO_OK) return rc;
    }
  }
  return flush();
}

template <typename F>
static int mt_apply(const char *what, void *const *const (&lists)[F::NL], const int64_t *sizes,
                    int64_t ntensors, const F &f, hipStream_t st) {
  constexpr int64_t kPiece = (int64_t)kMtThreads * kMtUnroll * F::E;
  return mt_for_each_table<F::NL>(what, lists, sizes, ntensors, kPiece,
                                  [&](const MtTable<F::NL> &tab, int64_t blocks) -> int {
                                    if (blocks == 0) return OSLO_OK;
                                    multi_tensor_apply_kernel<F>
                                        <<<dim3((unsigned)blocks), kMtThreads, 0, st>>>(tab, f);
                                    return check_launch(what);
                                  });
}

template <typename T> static int64_t norm_piece() {
  return (int64_t)kMtThreads * kMtUnroll * io<T>::EPV * kNormLoops;
}

static int64_t norm_piece_of(int dtype) {
  return dtype == OSLO_DTYPE_F32 ? norm_piece<float>() : norm_piece<__bf16>();
}

template <typename T, bool MAXNORM>
static int launch_norm(const void *const *x, const int64_t *sizes, int64_t ntensors, float *partials,
                       int64_t partials_len, float *out_global, float *out_per_tensor, int blend,
                       float alpha, float beta, int *noop, int skip_if_flag, hipStream_t st) {
  void *const *const lists[1] = {const_cast<void *const *>(x)};
  int64_t total = 0;
  const int rc = mt_for_each_table<1>(
      "multi_tensor_norm", lists, sizes, ntensors, norm_piece<T>(),
      [&](const MtTable<1> &tab, int64_t blocks) -> int {
        if (tab.block0 + blocks > partials_len)
          return fail(OSLO_ERR_WORKSPACE, "multi_tensor_norm: workspace of %lld values, %lld needed",
                      (long long)partials_len, (long long)(tab.block0 + blocks));
        if (blocks > 0) {
          multi_tensor_norm_kernel<T, MAXNORM>
              <<<dim3((unsigned)blocks), kMtThreads, 0, st>>>(tab, partials, noop, skip_if_flag);
          const int rc1 = check_launch("multi_tensor_norm_kernel");
          if (rc1 != OSLO_OK) return rc1;
        }
        if (out_per_tensor != nullptr) {
          multi_tensor_norm_finalize_kernel<MAXNORM>
              <<<dim3((unsigned)tab.ntensors), kMtThreads, 0, st>>>(tab, partials, out_per_tensor, blend,
                                                                    alpha, beta, noop, skip_if_flag);
          const int rc2 = check_launch("multi_tensor_norm_finalize_kernel");
          if (rc2 != OSLO_OK) return rc2;
        }
        total = tab.block0 + blocks;
        return OSLO_OK;
      });
  if (rc != OSLO_OK) return rc;
  if (out_global != nullptr) {
    multi_tensor_norm_global_kernel<MAXNORM><<<dim3(1), 1024, 0, st>>>(partials, total, out_global, noop,
                                                                       skip_if_flag);
    return check_launch("multi_tensor_norm_global_kernel");
  }
  return OSLO_OK;
}

static void bias_corrections(float beta1, float beta2, int step, int bias_correction, float *bc1,
                             float *bc2) {
  // std::pow on the float betas promotes to double; the result is stored as float
  *bc1 = 1.0f;
  *bc2 = 1.0f;
  if (bias_correction == 1) {
    *bc1 = (float)(1.0 - pow((double)beta1, (double)step));
    *bc2 = (float)(1.0 - pow((double)beta2, (double)step));
  }
}

}  // namespace oslo

extern "C" {

int oslo_multi_tensor_sgd(const void *const *g, void *const *w, void *const *mom,
                          void *const *w_copy, const int64_t *sizes, int64_t ntensors,
                          float weight_decay, float momentum, float dampening, float lr,
                          int nesterov, int first_run, int wd_after_momentum, float scale,
                          int dtype_grad, int dtype_weight, int dtype_copy, const int *noop_flag,
                          void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype_grad) || !valid_dtype(dtype_weight))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_sgd: unknown dtype %d / %d", dtype_grad,
                dtype_weight);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_sgd: negative tensor count");
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(g && w && mom && sizes, "multi_tensor_sgd: null table pointer");
  const bool copy = w_copy != nullptr;
  OSLO_REQUIRE(dtype_grad == dtype_weight || dtype_weight == OSLO_DTYPE_F32,
               "multi_tensor_sgd: gradients of dtype %d with weights of dtype %d (the weights must "
               "have the gradients' type or be float32)",
               dtype_grad, dtype_weight);
  OSLO_REQUIRE(!copy || (dtype_weight == OSLO_DTYPE_F32 &&
                         (dtype_copy == OSLO_DTYPE_F16 || dtype_copy == OSLO_DTYPE_BF16)),
               "multi_tensor_sgd: the extra output is a 16-bit copy of float32 weights");
  hipStream_t st = (hipStream_t)stream;
#define OSLO_SGD(TG_, TW_, TO_, OUT_)                                                          \
  do {                                                                                         \
    SgdOp<TG_, TW_, TO_, OUT_> f;                                                              \
    f.wd = weight_decay; f.momentum = momentum; f.dampening = dampening; f.lr = lr;            \
    f.scale = scale; f.nesterov = nesterov; f.first_run = first_run;                           \
    f.wd_after_momentum = wd_after_momentum; f.noop = noop_flag;                               \
    void *const *const lists[OUT_ ? 4 : 3] = {const_cast<void *const *>(g), w, mom OSLO_SGD_COPY_##OUT_}; \
    return mt_apply("multi_tensor_sgd", lists, sizes, ntensors, f, st);                        \
  } while (0)
#define OSLO_SGD_COPY_true , w_copy
#define OSLO_SGD_COPY_false
  if (!copy) {
    if (dtype_weight == OSLO_DTYPE_F32) {
      if (dtype_grad == OSLO_DTYPE_F32) OSLO_SGD(float, float, _Float16, false);
      if (dtype_grad == OSLO_DTYPE_F16) OSLO_SGD(_Float16, float, _Float16, false);
      OSLO_SGD(__bf16, float, _Float16, false);
    }
    if (dtype_weight == OSLO_DTYPE_F16) OSLO_SGD(_Float16, _Float16, _Float16, false);
    OSLO_SGD(__bf16, __bf16, _Float16, false);
  }
  if (dtype_copy == OSLO_DTYPE_F16) {
    if (dtype_grad == OSLO_DTYPE_F32) OSLO_SGD(float, float, _Float16, true);
    if (dtype_grad == OSLO_DTYPE_F16) OSLO_SGD(_Float16, float, _Float16, true);
    OSLO_SGD(__bf16, float, _Float16, true);
  }
  if (dtype_grad == OSLO_DTYPE_F32) OSLO_SGD(float, float, __bf16, true);
  if (dtype_grad == OSLO_DTYPE_F16) OSLO_SGD(_Float16, float, __bf16, true);
  OSLO_SGD(__bf16, float, __bf16, true);
#undef OSLO_SGD
#undef OSLO_SGD_COPY_true
#undef OSLO_SGD_COPY_false
}

int oslo_multi_tensor_adagrad(const void *const *g, void *const *p, void *const *h,
                              const int64_t *sizes, int64_t ntensors, float lr, float eps, int mode,
                              float weight_decay, int dtype, void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_adagrad: unknown dtype %d", dtype);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_adagrad: negative tensor count");
  OSLO_REQUIRE(mode == 0 || mode == 1, "multi_tensor_adagrad: mode %d is neither 0 (L2) nor 1 (decoupled)",
               mode);
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(g && p && h && sizes, "multi_tensor_adagrad: null table pointer");
  void *const *const lists[3] = {const_cast<void *const *>(g), p, h};
  hipStream_t st = (hipStream_t)stream;
#define OSLO_ADAGRAD(T_)                                                  \
  do {                                                                    \
    AdagradOp<T_> f;                                                      \
    f.eps = eps; f.lr = lr; f.decay = weight_decay; f.mode = mode;        \
    return mt_apply("multi_tensor_adagrad", lists, sizes, ntensors, f, st); \
  } while (0)
  if (dtype == OSLO_DTYPE_F32) OSLO_ADAGRAD(float);
  if (dtype == OSLO_DTYPE_F16) OSLO_ADAGRAD(_Float16);
  OSLO_ADAGRAD(__bf16);
#undef OSLO_ADAGRAD
}

int oslo_multi_tensor_novograd(const void *const *g, void *const *p, void *const *m,
                               const int64_t *sizes, int64_t ntensors, const float *grad_norms,
                               float lr, float beta1, float beta2, float eps, int step,
                               int bias_correction, float weight_decay, int grad_averaging,
                               int moment_mode, int dtype, void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_novograd: unknown dtype %d", dtype);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_novograd: negative tensor count");
  OSLO_REQUIRE(moment_mode == 0 || moment_mode == 1, "multi_tensor_novograd: moment mode %d", moment_mode);
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(g && p && m && sizes && grad_norms, "multi_tensor_novograd: null pointer");
  void *const *const lists[3] = {const_cast<void *const *>(g), p, m};
  hipStream_t st = (hipStream_t)stream;
  // multi_tensor_novograd.cu:118-129: the second correction is a square root
  // (the stored second moment is a norm, not its square)
  float bc1 = 1.0f, bc2 = 1.0f;
  if (bias_correction == 1) {
    bc1 = (float)(1.0 - pow((double)beta1, (double)step));
    bc2 = (float)sqrt(1.0 - pow((double)beta2, (double)step));
  }
#define OSLO_NOVOGRAD(T_)                                                                \
  do {                                                                                   \
    NovogradOp<T_> f;                                                                    \
    f.beta1 = beta1; f.beta3 = grad_averaging == 1 ? 1.f - beta1 : 1.f; f.bc1 = bc1;     \
    f.bc2 = bc2; f.eps = eps; f.lr = lr; f.decay = weight_decay;                         \
    f.moment_mode = moment_mode; f.grad_norms = grad_norms;                              \
    return mt_apply("multi_tensor_novograd", lists, sizes, ntensors, f, st);             \
  } while (0)
  if (dtype == OSLO_DTYPE_F32) OSLO_NOVOGRAD(float);
  if (dtype == OSLO_DTYPE_F16) OSLO_NOVOGRAD(_Float16);
  OSLO_NOVOGRAD(__bf16);
#undef OSLO_NOVOGRAD
}

int oslo_multi_tensor_lamb_stage1(void *const *g, const void *const *p, void *const *m,
                                  void *const *v, const int64_t *sizes, int64_t ntensors,
                                  float beta1, float beta2, float eps, int step, int bias_correction,
                                  float weight_decay, int grad_averaging, int mode,
                                  const float *global_grad_norm, float max_grad_norm, int dtype,
                                  void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_lamb_stage1: unknown dtype %d", dtype);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_lamb_stage1: negative tensor count");
  OSLO_REQUIRE(mode == 0 || mode == 1, "multi_tensor_lamb_stage1: mode %d is neither 0 (L2) nor 1 (decoupled)",
               mode);
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(g && p && m && v && sizes && global_grad_norm, "multi_tensor_lamb_stage1: null pointer");
  void *const *const lists[4] = {g, const_cast<void *const *>(p), m, v};
  hipStream_t st = (hipStream_t)stream;
  float bc1, bc2;
  bias_corrections(beta1, beta2, step, bias_correction, &bc1, &bc2);
#define OSLO_LAMB1(T_)                                                                     \
  do {                                                                                     \
    LambStage1Op<T_> f;                                                                    \
    f.beta1 = beta1; f.beta2 = beta2; f.beta3 = grad_averaging == 1 ? 1.f - beta1 : 1.f;   \
    f.bc1 = bc1; f.bc2 = bc2; f.eps = eps; f.decay = weight_decay;                         \
    f.max_global_grad_norm = max_grad_norm; f.mode = mode;                                 \
    f.global_grad_norm = global_grad_norm;                                                 \
    return mt_apply("multi_tensor_lamb_stage1", lists, sizes, ntensors, f, st);            \
  } while (0)
  if (dtype == OSLO_DTYPE_F32) OSLO_LAMB1(float);
  if (dtype == OSLO_DTYPE_F16) OSLO_LAMB1(_Float16);
  OSLO_LAMB1(__bf16);
#undef OSLO_LAMB1
}

int oslo_multi_tensor_lamb_stage2(const void *const *update, void *const *p, const int64_t *sizes,
                                  int64_t ntensors, const float *param_norms,
                                  const float *update_norms, float lr, float weight_decay,
                                  int use_nvlamb, int dtype, void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_lamb_stage2: unknown dtype %d", dtype);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_lamb_stage2: negative tensor count");
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(update && p && sizes && param_norms && update_norms, "multi_tensor_lamb_stage2: null pointer");
  void *const *const lists[2] = {const_cast<void *const *>(update), p};
  hipStream_t st = (hipStream_t)stream;
#define OSLO_LAMB2(T_)                                                           \
  do {                                                                           \
    LambStage2Op<T_> f;                                                          \
    f.lr = lr; f.decay = weight_decay; f.use_nvlamb = use_nvlamb;                \
    f.param_norms = param_norms; f.update_norms = update_norms;                  \
    return mt_apply("multi_tensor_lamb_stage2", lists, sizes, ntensors, f, st);  \
  } while (0)
  if (dtype == OSLO_DTYPE_F32) OSLO_LAMB2(float);
  if (dtype == OSLO_DTYPE_F16) OSLO_LAMB2(_Float16);
  OSLO_LAMB2(__bf16);
#undef OSLO_LAMB2
}

int oslo_multi_tensor_lamb_mp_stage1(void *const *g, const void *const *p, void *const *m,
                                     void *const *v, const int64_t *sizes, int64_t ntensors,
                                     float beta1, float beta2, float eps, const int *step,
                                     int bias_correction, float weight_decay, int grad_averaging,
                                     int mode, const float *global_grad_norm,
                                     const float *max_grad_norm, const float *inv_scale,
                                     const int *noop_flag, int dtype_grad, int dtype_param,
                                     void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype_grad) || !valid_dtype(dtype_param))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_lamb_mp_stage1: unknown dtype %d / %d", dtype_grad,
                dtype_param);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_lamb_mp_stage1: negative tensor count");
  OSLO_REQUIRE(mode == 0 || mode == 1, "multi_tensor_lamb_mp_stage1: mode %d is neither 0 (L2) nor 1 (decoupled)",
               mode);
  OSLO_REQUIRE(dtype_param == dtype_grad || dtype_param == OSLO_DTYPE_F32,
               "multi_tensor_lamb_mp_stage1: gradients of dtype %d with parameters of dtype %d (the "
               "parameters must have the gradients' type or be float32)",
               dtype_grad, dtype_param);
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(g && p && m && v && sizes && step && global_grad_norm && max_grad_norm && inv_scale,
               "multi_tensor_lamb_mp_stage1: null pointer");
  void *const *const lists[4] = {g, const_cast<void *const *>(p), m, v};
  hipStream_t st = (hipStream_t)stream;
#define OSLO_LAMB_MP1(TG_, TP_)                                                            \
  do {                                                                                     \
    LambMpStage1Op<TG_, TP_> f;                                                            \
    f.beta1 = beta1; f.beta2 = beta2; f.beta3 = grad_averaging == 1 ? 1.f - beta1 : 1.f;   \
    f.eps = eps; f.decay = weight_decay; f.mode = mode; f.bias_correction = bias_correction; \
    f.step = step; f.noop = noop_flag; f.global_grad_norm = global_grad_norm;              \
    f.max_global_grad_norm = max_grad_norm; f.inv_scale = inv_scale;                       \
    return mt_apply("multi_tensor_lamb_mp_stage1", lists, sizes, ntensors, f, st);         \
  } while (0)
  if (dtype_param == OSLO_DTYPE_F32) {
    if (dtype_grad == OSLO_DTYPE_F32) OSLO_LAMB_MP1(float, float);
    if (dtype_grad == OSLO_DTYPE_F16) OSLO_LAMB_MP1(_Float16, float);
    OSLO_LAMB_MP1(__bf16, float);
  }
  if (dtype_param == OSLO_DTYPE_F16) OSLO_LAMB_MP1(_Float16, _Float16);
  OSLO_LAMB_MP1(__bf16, __bf16);
#undef OSLO_LAMB_MP1
}

int oslo_multi_tensor_lamb_mp_stage2(const void *const *update, void *const *p, void *const *p_copy,
                                     const int64_t *sizes, int64_t ntensors,
                                     const float *param_norms, const float *update_norms,
                                     const float *lr, float weight_decay, int use_nvlamb,
                                     const int *noop_flag, int dtype_update, int dtype_param,
                                     void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype_update) || !valid_dtype(dtype_param))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_lamb_mp_stage2: unknown dtype %d / %d",
                dtype_update, dtype_param);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_lamb_mp_stage2: negative tensor count");
  const bool copy = p_copy != nullptr;
  OSLO_REQUIRE(copy ? dtype_param == OSLO_DTYPE_F32 : dtype_param == dtype_update,
               "multi_tensor_lamb_mp_stage2: update of dtype %d with parameters of dtype %d (one type, or "
               "float32 parameters with a copy in the update's type)",
               dtype_update, dtype_param);
  if (ntensors == 0) return OSLO_OK;
  OSLO_REQUIRE(update && p && sizes && param_norms && update_norms && lr,
               "multi_tensor_lamb_mp_stage2: null pointer");
  hipStream_t st = (hipStream_t)stream;
#define OSLO_LAMB_MP2(T_, TP_, OUT_)                                                       \
  do {                                                                                     \
    LambMpStage2Op<T_, TP_, OUT_> f;                                                       \
    f.decay = weight_decay; f.use_nvlamb = use_nvlamb; f.lr = lr;                          \
    f.param_norms = param_norms; f.update_norms = update_norms; f.noop = noop_flag;        \
    void *const *const lists[OUT_ ? 3 : 2] = {const_cast<void *const *>(update), p OSLO_LAMB_MP2_COPY_##OUT_}; \
    return mt_apply("multi_tensor_lamb_mp_stage2", lists, sizes, ntensors, f, st);         \
  } while (0)
#define OSLO_LAMB_MP2_COPY_true , p_copy
#define OSLO_LAMB_MP2_COPY_false
  if (copy) {
    if (dtype_update == OSLO_DTYPE_F32) OSLO_LAMB_MP2(float, float, true);
    if (dtype_update == OSLO_DTYPE_F16) OSLO_LAMB_MP2(_Float16, float, true);
    OSLO_LAMB_MP2(__bf16, float, true);
  }
  if (dtype_update == OSLO_DTYPE_F32) OSLO_LAMB_MP2(float, float, false);
  if (dtype_update == OSLO_DTYPE_F16) OSLO_LAMB_MP2(_Float16, _Float16, false);
  OSLO_LAMB_MP2(__bf16, __bf16, false);
#undef OSLO_LAMB_MP2
#undef OSLO_LAMB_MP2_COPY_true
#undef OSLO_LAMB_MP2_COPY_false
}

int64_t oslo_multi_tensor_norm_partials(const int64_t *sizes, int64_t ntensors, int dtype) {
  using namespace oslo;
  if (!valid_dtype(dtype) || ntensors < 0 || (ntensors > 0 && sizes == nullptr)) {
    fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_norm_partials: bad arguments");
    return OSLO_ERR_INVALID_ARGUMENT;
  }
  int64_t total = 0;
  for (int64_t i = 0; i < ntensors; ++i) {
    if (sizes[i] < 0) {
      fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_norm_partials: tensor %lld has size %lld",
           (long long)i, (long long)sizes[i]);
      return OSLO_ERR_INVALID_ARGUMENT;
    }
    total += ceil_div(sizes[i], norm_piece_of(dtype));
  }
  return total > 0 ? total : 1;
}

int oslo_multi_tensor_norm(const void *const *x, const int64_t *sizes, int64_t ntensors, int dtype,
                           float *partials, int64_t partials_len, float *out_global,
                           float *out_per_tensor, int norm_type, int blend, float alpha, float beta,
                           int *noop_flag, int skip_if_flag, void *stream) {
  using namespace oslo;
  tune_snapshot();
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "multi_tensor_norm: unknown dtype %d", dtype);
  OSLO_REQUIRE(ntensors >= 0, "multi_tensor_norm: negative tensor count");
  OSLO_REQUIRE(norm_type == 0 || norm_type == 2, "multi_tensor_norm: norm type %d is neither 2 (L2) nor 0 (max)",
               norm_type);
  OSLO_REQUIRE(blend == 0 || out_per_tensor != nullptr, "multi_tensor_norm: blending needs the per-tensor output");
  OSLO_REQUIRE(partials != nullptr && partials_len >= 1, "multi_tensor_norm: no workspace");
  OSLO_REQUIRE(!skip_if_flag || noop_flag != nullptr, "multi_tensor_norm: skip_if_flag without a flag");
  OSLO_REQUIRE(ntensors == 0 || (x && sizes), "multi_tensor_norm: null table pointer");
  hipStream_t st = (hipStream_t)stream;
#define OSLO_NORM(T_)                                                                               \
  (norm_type == 0 ? launch_norm<T_, true>(x, sizes, ntensors, partials, partials_len, out_global,   \
                                          out_per_tensor, blend, alpha, beta, noop_flag,            \
                                          skip_if_flag, st)                                         \
                  : launch_norm<T_, false>(x, sizes, ntensors, partials, partials_len, out_global,  \
                                           out_per_tensor, blend, alpha, beta, noop_flag,           \
                                           skip_if_flag, st))
  if (dtype == OSLO_DTYPE_F32) return OSLO_NORM(float);
  if (dtype == OSLO_DTYPE_F16) return OSLO_NORM(_Float16);
  return OSLO_NORM(__bf16);
#undef OSLO_NORM
}

}  // extern "C"
