// LayerNorm / RMSNorm in double precision for gfx950.
//
// The reference's forward dispatch admits double tensors
// (oslo/torch/_C/csrc/fused_layer_norm.cu:780, 799, with U = double for the
// statistics, oslo/torch/_C/csrc/includes/type_shim.h:172-186), and so does its
// RMS backward (fused_layer_norm.cu:950).  Double rows are a debugging and
// gradient-checking format, not a throughput one: these kernels are plain
// (one 256-lane workgroup per row, two passes over the row, scalar 8-byte
// accesses), accumulate in double and keep mean and invvar in double.  The
// backward is offered for both norms.
#include <math.h>

#include "capi.h"

namespace oslo {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

// Sum over the workgroup; every lane receives the total.  `red` has kWaves
// slots and may be reused by the next call.
__device__ __forceinline__ double block_sum_f64(double v, double *red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();  // readers of the previous call are done with red[]
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  double t = red[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) t += red[w];
  return t;
}

// y = gamma * ((x - mean) * invvar) + beta, fused_layer_norm.cu:322-349 with
// every type double.
template <bool RMS>
__global__ __launch_bounds__(kThreads) void norm_f64_fwd_kernel(
    const double *__restrict__ x, const double *__restrict__ gamma,
    const double *__restrict__ beta, double *__restrict__ y,
    double *__restrict__ mean, double *__restrict__ invvar, int64_t n1,
    int64_t n2, double eps) {
  __shared__ double red[kWaves];
  for (int64_t row = blockIdx.x; row < n1; row += gridDim.x) {
    const double *xr = x + row * n2;
    double *yr = y + row * n2;
    double mu = 0.0;
    if (!RMS) {
      double s = 0.0;
      for (int64_t j = threadIdx.x; j < n2; j += kThreads) s += xr[j];
      mu = block_sum_f64(s, red) / (double)n2;
    }
    double q = 0.0;
    for (int64_t j = threadIdx.x; j < n2; j += kThreads) {
      const double d = xr[j] - mu;
      q += d * d;
    }
    const double var = block_sum_f64(q, red) / (double)n2;
    const double iv = 1.0 / sqrt(var + eps);
    for (int64_t j = threadIdx.x; j < n2; j += kThreads) {
      double v = (xr[j] - mu) * iv;
      if (gamma != nullptr) {
        v = gamma[j] * v;
        if (!RMS) v += beta[j];
      }
      yr[j] = v;
    }
    if (threadIdx.x == 0) {
      if (!RMS) mean[row] = mu;
      invvar[row] = iv;
    }
  }
}

// grad_input of fused_layer_norm.cu:594-741 with every type double.
template <bool RMS>
__global__ __launch_bounds__(kThreads) void norm_f64_bwd_dx_kernel(
    const double *__restrict__ dy, const double *__restrict__ x,
    const double *__restrict__ mean, const double *__restrict__ invvar,
    const double *__restrict__ gamma, double *__restrict__ dx, int64_t n1,
    int64_t n2) {
  __shared__ double red[kWaves];
  for (int64_t row = blockIdx.x; row < n1; row += gridDim.x) {
    const double *gr = dy + row * n2;
    const double *xr = x + row * n2;
    double *dr = dx + row * n2;
    const double mu = RMS ? 0.0 : mean[row];
    const double iv = invvar[row];
    double s1 = 0.0, s2 = 0.0;
    for (int64_t j = threadIdx.x; j < n2; j += kThreads) {
      const double dg = gamma != nullptr ? gr[j] * gamma[j] : gr[j];
      if (!RMS) s1 += dg;
      s2 += dg * (xr[j] - mu) * iv;
    }
    if (!RMS) s1 = block_sum_f64(s1, red);
    s2 = block_sum_f64(s2, red);
    const double fh = (double)n2;
    const double term = iv / fh;
    for (int64_t j = threadIdx.x; j < n2; j += kThreads) {
      const double dg = gamma != nullptr ? gr[j] * gamma[j] : gr[j];
      double f = fh * dg;
      if (!RMS) f -= s1;
      f -= (xr[j] - mu) * iv * s2;
      dr[j] = f * term;
    }
  }
}

// dgamma[j] = sum over rows of dy * xhat, dbeta[j] = sum over rows of dy
// (fused_layer_norm.cu:458-591).  64 columns per workgroup, four row lanes.
template <bool RMS>
__global__ __launch_bounds__(kThreads) void norm_f64_bwd_param_kernel(
    const double *__restrict__ dy, const double *__restrict__ x,
    const double *__restrict__ mean, const double *__restrict__ invvar,
    double *__restrict__ dgamma, double *__restrict__ dbeta, int64_t n1,
    int64_t n2) {
  __shared__ double sg[kWaves][64];
  __shared__ double sb[kWaves][64];
  const int cx = threadIdx.x & 63;
  const int ry = threadIdx.x >> 6;
  const int64_t col = (int64_t)blockIdx.x * 64 + cx;
  double ag = 0.0, ab = 0.0;
  if (col < n2) {
    for (int64_t r = ry; r < n1; r += kWaves) {
      const double g = dy[r * n2 + col];
      const double mu = RMS ? 0.0 : mean[r];
      ag += g * (x[r * n2 + col] - mu) * invvar[r];
      ab += g;
    }
  }
  sg[ry][cx] = ag;
  sb[ry][cx] = ab;
  __syncthreads();
  if (ry == 0 && col < n2) {
    double tg = sg[0][cx], tb = sb[0][cx];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      tg += sg[w][cx];
      tb += sb[w][cx];
    }
    dgamma[col] = tg;
    if (!RMS) dbeta[col] = tb;
  }
}

unsigned row_grid(int64_t n1) { return (unsigned)(n1 < 65536 ? n1 : 65536); }

}  // namespace

int launch_norm_f64_fwd(bool rms, const void *x, const void *gamma,
                        const void *beta, void *y, void *mean, void *invvar,
                        int64_t n1, int64_t n2, double eps, hipStream_t st) {
  const dim3 grid(row_grid(n1));
  if (rms)
    norm_f64_fwd_kernel<true><<<grid, kThreads, 0, st>>>(
        (const double *)x, (const double *)gamma, nullptr, (double *)y, nullptr,
        (double *)invvar, n1, n2, eps);
  else
    norm_f64_fwd_kernel<false><<<grid, kThreads, 0, st>>>(
        (const double *)x, (const double *)gamma, (const double *)beta,
        (double *)y, (double *)mean, (double *)invvar, n1, n2, eps);
  return check_launch("norm_f64_fwd_kernel");
}

int launch_norm_f64_bwd(bool rms, const void *dy, const void *x,
                        const void *mean, const void *invvar,
                        const void *gamma, void *dx, void *dgamma, void *dbeta,
                        int64_t n1, int64_t n2, hipStream_t st) {
  const dim3 grid(row_grid(n1));
  if (rms)
    norm_f64_bwd_dx_kernel<true><<<grid, kThreads, 0, st>>>(
        (const double *)dy, (const double *)x, nullptr, (const double *)invvar,
        (const double *)gamma, (double *)dx, n1, n2);
  else
    norm_f64_bwd_dx_kernel<false><<<grid, kThreads, 0, st>>>(
        (const double *)dy, (const double *)x, (const double *)mean,
        (const double *)invvar, (const double *)gamma, (double *)dx, n1, n2);
  int rc = check_launch("norm_f64_bwd_dx_kernel");
  if (rc != OSLO_OK || dgamma == nullptr) return rc;
  const dim3 pgrid((unsigned)ceil_div(n2, 64));
  if (rms)
    norm_f64_bwd_param_kernel<true><<<pgrid, kThreads, 0, st>>>(
        (const double *)dy, (const double *)x, nullptr, (const double *)invvar,
        (double *)dgamma, nullptr, n1, n2);
  else
    norm_f64_bwd_param_kernel<false><<<pgrid, kThreads, 0, st>>>(
        (const double *)dy, (const double *)x, (const double *)mean,
        (const double *)invvar, (double *)dgamma, (double *)dbeta, n1, n2);
  return check_launch("norm_f64_bwd_param_kernel");
}

}  // namespace oslo
