// Deterministic reduction of fp32 column-partial rows to a parameter gradient,
// shared by the norm, bias-GeLU and bias-dropout-add backward passes.
#pragma once

#include "capi.h"
#include "common.hip.h"

namespace oslo {

// Reduces fp32 partial rows part[a][0..P)[cols] to out_a[cols] in dtype V;
// blockIdx.y selects the array a (up to three; a null output is skipped).
// A workgroup owns CQ column quads (CQ * 4 columns) times SL slices of the
// partial rows (CQ * SL threads), so that for the usual P of a few hundred
// every thread issues all its loads at once; the slices are then folded
// through LDS in a fixed order.  cols % 4 == 0.
template <typename V, int SL, int CQ>
__global__ __launch_bounds__(SL * CQ) void colsum_finalize_kernel(
    const float *__restrict__ part, int64_t P, int64_t cols,
    V *__restrict__ out0, V *__restrict__ out1, V *__restrict__ out2) {
  constexpr int C = CQ * 4;  // columns of a workgroup
  static_assert(SL % 8 == 0 && C * 8 <= SL * CQ, "the second fold uses 8 * C threads");
  __shared__ float sh[SL][C + 1];
  __shared__ float sh2[8][C + 1];
  const int tid = threadIdx.x;
  const int cq = tid % CQ, ps = tid / CQ;
  const int64_t col = ((int64_t)blockIdx.x * CQ + cq) * 4;
  const int a = blockIdx.y;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (col < cols) {
    const float *base = part + (int64_t)a * P * cols + col;
#pragma unroll 4
    for (int64_t p = ps; p < P; p += SL) {
      float t[4];
      io<float>::unpack(ld16_cached(base + p * cols), t);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += t[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) sh[ps][cq * 4 + e] = acc[e];
  __syncthreads();
  if (tid < 8 * C) {
    const int g = tid / C, c = tid % C;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < SL / 8; ++i) s += sh[g * (SL / 8) + i][c];
    sh2[g][c] = s;
  }
  __syncthreads();
  if (tid < C) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < 8; ++g) s += sh2[g][tid];
    const int64_t oc = (int64_t)blockIdx.x * C + tid;
    V *o = a == 0 ? out0 : (a == 1 ? out1 : out2);
    if (oc < cols && o != nullptr) o[oc] = io<V>::to_scalar(s);
  }
}

template <typename V>
static inline int launch_colsum_finalize(const float *part, int64_t P,
                                         int64_t cols, void *out0, void *out1,
                                         hipStream_t st, void *out2 = nullptr,
                                         int narrays = 0) {
  // narrays = number of arrays of partial rows (outputs that are null are
  // skipped); by default one per non-null output
  if (narrays <= 0) narrays = out1 != nullptr ? 2 : 1;
  const int slices = g_tune.colsum_slices > 0 ? g_tune.colsum_slices : 128;
  if (slices == 256) {
    const dim3 blocks((unsigned)ceil_div(cols, 16), (unsigned)narrays);
    colsum_finalize_kernel<V, 256, 4><<<blocks, 1024, 0, st>>>(
        part, P, cols, (V *)out0, (V *)out1, (V *)out2);
  } else if (slices == 64) {
    const dim3 blocks((unsigned)ceil_div(cols, 32), (unsigned)narrays);
    colsum_finalize_kernel<V, 64, 8><<<blocks, 512, 0, st>>>(
        part, P, cols, (V *)out0, (V *)out1, (V *)out2);
  } else {
    const dim3 blocks((unsigned)ceil_div(cols, 32), (unsigned)narrays);
    colsum_finalize_kernel<V, 128, 8><<<blocks, 1024, 0, st>>>(
        part, P, cols, (V *)out0, (V *)out1, (V *)out2);
  }
  return check_launch("colsum_finalize_kernel");
}

// ---------------------------------------------------------------------------
// Column sums on the generic path (any column count, any alignment), in two
// steps: S slices of the rows are summed side by side into fp32 partial rows,
// then one thread per column adds the S partials in a fixed order.
// ---------------------------------------------------------------------------

// f(row, col, acc) adds the contributions of element (row, col) to acc[0..NA).
// grid = (ceil(cols / 64), S); a workgroup is 64 columns x 4 row lanes.
template <int NA, typename F>
__global__ __launch_bounds__(256) void colpart_generic_kernel(
    F f, float *__restrict__ part, int64_t rows, int64_t cols) {
  __shared__ float sh[NA][4][64];
  const int cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
  const int64_t col = (int64_t)blockIdx.x * 64 + cx;
  const int64_t S = gridDim.y, slice = blockIdx.y;
  float acc[NA];
#pragma unroll
  for (int a = 0; a < NA; ++a) acc[a] = 0.f;
  if (col < cols)
    for (int64_t r = slice * 4 + ry; r < rows; r += S * 4) f(r, col, acc);
#pragma unroll
  for (int a = 0; a < NA; ++a) sh[a][ry][cx] = acc[a];
  __syncthreads();
  if (ry == 0 && col < cols) {
#pragma unroll
    for (int a = 0; a < NA; ++a)
      part[((int64_t)a * S + slice) * cols + col] =
          (sh[a][0][cx] + sh[a][1][cx]) + (sh[a][2][cx] + sh[a][3][cx]);
  }
}

// grid = (ceil(cols / 256), arrays); a null output is skipped.
template <typename V>
__global__ __launch_bounds__(256) void colfinal_generic_kernel(
    const float *__restrict__ part, int64_t S, int64_t cols,
    V *__restrict__ out0, V *__restrict__ out1) {
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int a = blockIdx.y;
  V *o = a == 0 ? out0 : out1;
  if (col >= cols || o == nullptr) return;
  float s = 0.f;
  for (int64_t p = 0; p < S; ++p) s += part[((int64_t)a * S + p) * cols + col];
  o[col] = io<V>::to_scalar(s);
}

// Row slices that fit a workspace of ws_bytes (0: the workspace cannot be
// used and the caller falls back to one thread per column).
static inline int64_t generic_colsum_slices(const void *ws, int64_t ws_bytes,
                                            int narrays, int64_t rows,
                                            int64_t cols) {
  if (ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 3u) != 0) return 0;
  int64_t S = ws_bytes / ((int64_t)narrays * cols * (int64_t)sizeof(float));
  const int64_t want = ceil_div(rows, 16);  // at least four steps per slice
  const int64_t cap = (int64_t)device_cu_count() * 4;
  if (S > want) S = want;
  if (S > cap) S = cap;
  if (S > 65535) S = 65535;
  return S < 1 ? 0 : S;
}

// Launches both steps.  NA arrays; out1 may be null when NA == 1.
template <int NA, typename V, typename F>
static inline int launch_generic_colsum(F f, void *ws, int64_t S, int64_t rows,
                                        int64_t cols, void *out0, void *out1,
                                        hipStream_t st) {
  colpart_generic_kernel<NA, F>
      <<<dim3((unsigned)ceil_div(cols, 64), (unsigned)S), 256, 0, st>>>(
          f, (float *)ws, rows, cols);
  int rc = check_launch("colpart_generic_kernel");
  if (rc != OSLO_OK) return rc;
  colfinal_generic_kernel<V>
      <<<dim3((unsigned)ceil_div(cols, 256), (unsigned)NA), 256, 0, st>>>(
          (const float *)ws, S, cols, (V *)out0, (V *)out1);
  return check_launch("colfinal_generic_kernel");
}

// Functor: the stored value itself (column sum of a [rows, cols] tensor).
template <typename T> struct StoredValue {
  const T *a;
  int64_t cols;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float *acc) const {
    acc[0] += io<T>::from_scalar(a[r * cols + c]);
  }
};

}  // namespace oslo
