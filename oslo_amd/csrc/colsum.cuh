// Deterministic reduction of fp32 column-partial rows to a parameter gradient,
// shared by the norm, bias-GeLU and bias-dropout-add backward passes.
#pragma once

#include "capi.h"
#include "common.cuh"

namespace oslo {

// Reduces fp32 partial rows part[a][0..P) [cols] (a < narr) to out_a[cols] in
// dtype V.  Workgroup = 8 column quads x 32 partial-row slices; cols % 4 == 0.
template <typename V>
__global__ __launch_bounds__(256) void colsum_finalize_kernel(
    const float *__restrict__ part, int64_t P, int64_t cols,
    V *__restrict__ out0, V *__restrict__ out1) {
  __shared__ float sh[32][33];
  const int tid = threadIdx.x;
  const int cq = tid & 7, ps = tid >> 3;
  const int64_t col = ((int64_t)blockIdx.x * 8 + cq) * 4;
  const int narr = out1 != nullptr ? 2 : 1;
  for (int a = 0; a < narr; ++a) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (col < cols) {
      const float *base = part + (int64_t)a * P * cols + col;
#pragma unroll 4
      for (int64_t p = ps; p < P; p += 32) {
        float t[4];
        io<float>::unpack(ld16_cached(base + p * cols), t);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += t[e];
      }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 4; ++e) sh[ps][cq * 4 + e] = acc[e];
    __syncthreads();
    if (tid < 32) {
      float s = 0.f;
#pragma unroll
      for (int p = 0; p < 32; ++p) s += sh[p][tid];
      const int64_t oc = (int64_t)blockIdx.x * 32 + tid;
      if (oc < cols) {
        V *o = a == 0 ? out0 : out1;
        o[oc] = io<V>::to_scalar(s);
      }
    }
  }
}

template <typename V>
static inline int launch_colsum_finalize(const float *part, int64_t P, int64_t cols,
                                  void *out0, void *out1, hipStream_t st) {
  const int64_t grid = ceil_div(cols, 32);
  colsum_finalize_kernel<V><<<dim3((unsigned)grid), 256, 0, st>>>(
      part, P, cols, (V *)out0, (V *)out1);
  return check_launch("colsum_finalize_kernel");
}

}  // namespace oslo
