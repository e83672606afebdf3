// A caller of liboslo_hip.so that knows nothing of Python or torch: plain HIP
// host code, the public header, hipMalloc'ed buffers and a stream of its own.
// It runs LayerNorm forward + backward (bf16 I/O) and the causal softmax
// forward (fp32) on small problems, checks them against double-precision loops
// written here, and exits non-zero on any mismatch or error code.  It is what
// a C or C++ host of the reference (a pybind module, an inference server) would
// do; the Python binding does the same through ctypes.
//
//   make -C oslo_amd/csrc c_abi_client && oslo_amd/csrc/c_abi_client
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/oslo_hip.h"

#define HIP_OK(call)                                                          \
  do {                                                                        \
    hipError_t e_ = (call);                                                   \
    if (e_ != hipSuccess) {                                                   \
      std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));         \
      std::exit(2);                                                           \
    }                                                                         \
  } while (0)

#define OSLO_CHECK(call)                                                      \
  do {                                                                        \
    int rc_ = (call);                                                         \
    if (rc_ != OSLO_OK) {                                                     \
      std::fprintf(stderr, "%s -> %d: %s\n", #call, rc_, oslo_hip_last_error()); \
      std::exit(3);                                                           \
    }                                                                         \
  } while (0)

static uint16_t to_bf16(float f) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// a small deterministic generator: the values only have to be varied
static float next_value(uint32_t &s) {
  s = s * 1664525u + 1013904223u;
  return ((float)((s >> 8) & 0xffff) / 32768.0f) - 1.0f;
}

template <typename T>
static T *to_device(const std::vector<T> &h) {
  T *d = nullptr;
  HIP_OK(hipMalloc(&d, h.size() * sizeof(T)));
  HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}
template <typename T>
static std::vector<T> to_host(const T *d, size_t n) {
  std::vector<T> h(n);
  HIP_OK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
  return h;
}

static int fails = 0;
static void expect_close(const char *what, double got, double want, double rel, double abs_) {
  if (!(std::fabs(got - want) <= rel * std::fabs(want) + abs_)) {
    if (fails < 10) std::fprintf(stderr, "%s: got %.8g, want %.8g\n", what, got, want);
    ++fails;
  }
}

static void layer_norm_bf16(hipStream_t st) {
  const int64_t n1 = 96, n2 = 1024;
  const double eps = 1e-5;
  uint32_t seed = 7;
  std::vector<uint16_t> x(n1 * n2), dy(n1 * n2), gamma(n2), beta(n2);
  for (auto &v : x) v = to_bf16(2.0f * next_value(seed));
  for (auto &v : dy) v = to_bf16(next_value(seed));
  for (auto &v : gamma) v = to_bf16(1.0f + 0.1f * next_value(seed));
  for (auto &v : beta) v = to_bf16(0.1f * next_value(seed));
  uint16_t *dx_ = to_device(x), *ddy = to_device(dy), *dg = to_device(gamma), *db = to_device(beta);
  uint16_t *y = nullptr, *dxo = nullptr, *dgamma = nullptr, *dbeta = nullptr;
  float *mean = nullptr, *invvar = nullptr;
  HIP_OK(hipMalloc(&y, n1 * n2 * 2));
  HIP_OK(hipMalloc(&dxo, n1 * n2 * 2));
  HIP_OK(hipMalloc(&dgamma, n2 * 2));
  HIP_OK(hipMalloc(&dbeta, n2 * 2));
  HIP_OK(hipMalloc(&mean, n1 * 4));
  HIP_OK(hipMalloc(&invvar, n1 * 4));
  // the caller owns the backward workspace: its size comes from the library
  const int64_t ws_bytes = oslo_workspace_bytes(OSLO_OP_LN_BWD, n1, n2);
  void *ws = nullptr;
  HIP_OK(hipMalloc(&ws, ws_bytes > 0 ? ws_bytes : 16));

  OSLO_CHECK(oslo_ln_fwd(dx_, dg, db, y, mean, invvar, n1, n2, eps, OSLO_DTYPE_BF16, OSLO_DTYPE_BF16, st));
  OSLO_CHECK(oslo_ln_bwd(ddy, dx_, mean, invvar, dg, dxo, dgamma, dbeta, ws, ws_bytes, n1, n2,
                         OSLO_DTYPE_BF16, OSLO_DTYPE_BF16, st));
  HIP_OK(hipStreamSynchronize(st));

  const auto hy = to_host(y, n1 * n2), hdx = to_host(dxo, n1 * n2);
  const auto hdg = to_host(dgamma, n2), hdb = to_host(dbeta, n2);
  std::vector<double> sum_dg(n2, 0.0), sum_db(n2, 0.0);
  for (int64_t r = 0; r < n1; ++r) {
    double m = 0, q = 0;
    for (int64_t c = 0; c < n2; ++c) m += from_bf16(x[r * n2 + c]);
    m /= n2;
    for (int64_t c = 0; c < n2; ++c) {
      const double d = from_bf16(x[r * n2 + c]) - m;
      q += d * d;
    }
    const double inv = 1.0 / std::sqrt(q / n2 + eps);
    double s1 = 0, s2 = 0;
    for (int64_t c = 0; c < n2; ++c) {
      const double xh = (from_bf16(x[r * n2 + c]) - m) * inv;
      const double g = from_bf16(dy[r * n2 + c]) * (double)from_bf16(gamma[c]);
      s1 += g;
      s2 += g * xh;
      sum_dg[c] += from_bf16(dy[r * n2 + c]) * xh;
      sum_db[c] += from_bf16(dy[r * n2 + c]);
    }
    for (int64_t c = 0; c < n2; ++c) {
      const double xh = (from_bf16(x[r * n2 + c]) - m) * inv;
      const double want_y = xh * from_bf16(gamma[c]) + from_bf16(beta[c]);
      const double g = from_bf16(dy[r * n2 + c]) * (double)from_bf16(gamma[c]);
      const double want_dx = inv / n2 * (n2 * g - s1 - xh * s2);
      // bf16 outputs: half an ulp is 2^-9 of the value
      expect_close("layer norm y", from_bf16(hy[r * n2 + c]), want_y, 1.0 / 256, 1e-3);
      expect_close("layer norm dx", from_bf16(hdx[r * n2 + c]), want_dx, 1.0 / 256, 2e-3);
    }
  }
  for (int64_t c = 0; c < n2; ++c) {
    expect_close("layer norm dgamma", from_bf16(hdg[c]), sum_dg[c], 1.0 / 128, 2e-2);
    expect_close("layer norm dbeta", from_bf16(hdb[c]), sum_db[c], 1.0 / 128, 2e-2);
  }
  for (void *p : {(void *)dx_, (void *)ddy, (void *)dg, (void *)db, (void *)y, (void *)dxo, (void *)dgamma,
                  (void *)dbeta, (void *)mean, (void *)invvar, ws})
    HIP_OK(hipFree(p));
}

static void causal_softmax_f32(hipStream_t st) {
  const int64_t batches = 5, sq = 40, sk = 64;
  const float scale = 0.25f;
  uint32_t seed = 11;
  std::vector<float> x(batches * sq * sk);
  for (auto &v : x) v = 4.0f * next_value(seed);
  float *dx = to_device(x), *y = nullptr;
  HIP_OK(hipMalloc(&y, x.size() * 4));
  OSLO_CHECK(oslo_softmax_causal_fwd(dx, y, batches, sq, sk, scale, OSLO_DTYPE_F32, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto hy = to_host(y, x.size());
  for (int64_t b = 0; b < batches; ++b)
    for (int64_t i = 0; i < sq; ++i) {
      const int64_t visible = i + 1 + (sk - sq);  // key j is visible when j <= i + (sk - sq)
      const float *xr = &x[(b * sq + i) * sk];
      double mx = -1e300, s = 0;
      for (int64_t j = 0; j < visible; ++j) mx = std::fmax(mx, (double)xr[j] * scale);
      for (int64_t j = 0; j < visible; ++j) s += std::exp((double)xr[j] * scale - mx);
      for (int64_t j = 0; j < sk; ++j) {
        const double want = j < visible ? std::exp((double)xr[j] * scale - mx) / s : 0.0;
        const double got = hy[(b * sq + i) * sk + j];
        if (j >= visible && got != 0.0) {
          std::fprintf(stderr, "causal softmax: a hidden key is not an exact zero\n");
          ++fails;
        }
        expect_close("causal softmax y", got, want, 1e-5, 1e-9);
      }
    }
  // errors are codes and messages, never exceptions or aborts
  if (oslo_softmax_causal_fwd(dx, y, batches, sq, sk, scale, 99, st) == OSLO_OK ||
      std::strlen(oslo_hip_last_error()) == 0) {
    std::fprintf(stderr, "an unknown dtype code was not refused\n");
    ++fails;
  }
  HIP_OK(hipFree(dx));
  HIP_OK(hipFree(y));
}

// softmax(scale * x + M) with the additive key mask [b, 1, 1, sk] of
// oslo/transformers/models/bert/modeling_bert.py:298-306 (-10000 on the
// padded keys) under the diagonal, forward and backward, float32
static void additive_mask_softmax_f32(hipStream_t st) {
  const int64_t b = 3, np = 2, sq = 24, sk = 32;
  const float scale = 0.5f;
  uint32_t seed = 23;
  std::vector<float> x(b * np * sq * sk), g(x.size()), m(b * sk, 0.f);
  for (auto &v : x) v = 4.0f * next_value(seed);
  for (auto &v : g) v = next_value(seed);
  const int64_t valid[3] = {32, 20, 9};
  for (int64_t i = 0; i < b; ++i)
    for (int64_t j = valid[i]; j < sk; ++j) m[i * sk + j] = -10000.f;
  float *dx_ = to_device(x), *dg = to_device(g), *dm = to_device(m), *y = nullptr, *dxo = nullptr;
  HIP_OK(hipMalloc(&y, x.size() * 4));
  HIP_OK(hipMalloc(&dxo, x.size() * 4));
  // the mask broadcasts over heads and queries: their strides are 0
  OSLO_CHECK(oslo_softmax_bias_fwd(dx_, dm, y, b, np, sq, sk, sk, 0, 0, OSLO_DTYPE_F32,
                                   OSLO_SOFTMAX_CAUSAL, scale, OSLO_DTYPE_F32, st));
  OSLO_CHECK(oslo_softmax_bias_bwd(dg, y, dm, dxo, b, np, sq, sk, sk, 0, 0, OSLO_DTYPE_F32,
                                   OSLO_SOFTMAX_CAUSAL | OSLO_SOFTMAX_SKIP_HIDDEN, scale,
                                   OSLO_DTYPE_F32, st));
  HIP_OK(hipStreamSynchronize(st));
  const auto hy = to_host(y, x.size());
  const auto hdx = to_host(dxo, x.size());
  for (int64_t r = 0; r < b * np * sq; ++r) {
    const int64_t bi = r / (np * sq), i = r % sq;
    const int64_t visible = i + 1 + (sk - sq);
    const float *xr = &x[r * sk];
    std::vector<double> u(sk), p(sk);
    double mx = -1e300, s = 0, dot = 0;
    for (int64_t j = 0; j < visible; ++j) {
      // the kernel forms the sum in float32 with one multiply-add
      u[j] = (double)std::fmaf(xr[j], scale, m[bi * sk + j]);
      mx = std::fmax(mx, u[j]);
    }
    for (int64_t j = 0; j < visible; ++j) s += std::exp(u[j] - mx);
    for (int64_t j = 0; j < sk; ++j) p[j] = j < visible ? std::exp(u[j] - mx) / s : 0.0;
    for (int64_t j = 0; j < sk; ++j) dot += p[j] * g[r * sk + j];
    for (int64_t j = 0; j < sk; ++j) {
      expect_close("additive-mask softmax y", hy[r * sk + j], p[j], 1e-5, 1e-9);
      if (j >= visible && hy[r * sk + j] != 0.0f) {
        std::fprintf(stderr, "additive-mask softmax: a key beyond the diagonal is not an exact zero\n");
        ++fails;
      }
      expect_close("additive-mask softmax dx", hdx[r * sk + j], scale * p[j] * (g[r * sk + j] - dot),
                   1e-5, 2e-7);
    }
  }
  // a term in a type the kernel does not add is refused with a message
  if (oslo_softmax_bias_fwd(dx_, dm, y, b, np, sq, sk, sk, 0, 0, OSLO_DTYPE_F16, 0, scale,
                            OSLO_DTYPE_F32, st) == OSLO_OK ||
      std::strlen(oslo_hip_last_error()) == 0) {
    std::fprintf(stderr, "a float16 term next to float32 scores was not refused\n");
    ++fails;
  }
  for (void *q : {(void *)dx_, (void *)dg, (void *)dm, (void *)y, (void *)dxo}) HIP_OK(hipFree(q));
}

int main() {
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  if (ndev == 0) {
    std::fprintf(stderr, "no GPU\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t st;
  HIP_OK(hipStreamCreate(&st));
  std::printf("liboslo_hip.so built for %s\n", oslo_hip_arch());
  layer_norm_bf16(st);
  causal_softmax_f32(st);
  additive_mask_softmax_f32(st);
  HIP_OK(hipStreamDestroy(st));
  if (fails) {
    std::fprintf(stderr, "%d mismatches\n", fails);
    return 1;
  }
  std::printf("c_abi_client: ok\n");
  return 0;
}
