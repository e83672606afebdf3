// Deterministic reduction of fp32 column-partial rows to a parameter gradient,
// shared by the norm, bias-GeLU and bias-dropout-add backward passes.
#pragma once

#include "capi.h"
#include "common.cuh"

namespace oslo {

// Reduces fp32 partial rows part[a][0..P)[cols] to out_a[cols] in dtype V;
// blockIdx.y selects the array a (up to three; a null output is skipped).
// A workgroup owns 32 columns: 8 column quads
// times 128 slices of the partial rows, so that for the usual P of a few
// hundred every thread issues all its loads at once; the slices are then
// folded through LDS in a fixed order.  cols % 4 == 0.
template <typename V>
__global__ __launch_bounds__(1024) void colsum_finalize_kernel(
    const float *__restrict__ part, int64_t P, int64_t cols,
    V *__restrict__ out0, V *__restrict__ out1, V *__restrict__ out2) {
  __shared__ float sh[128][33];
  __shared__ float sh2[8][33];
  const int tid = threadIdx.x;
  const int cq = tid & 7, ps = tid >> 3;
  const int64_t col = ((int64_t)blockIdx.x * 8 + cq) * 4;
  const int a = blockIdx.y;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (col < cols) {
    const float *base = part + (int64_t)a * P * cols + col;
#pragma unroll 4
    for (int64_t p = ps; p < P; p += 128) {
      float t[4];
      io<float>::unpack(ld16_cached(base + p * cols), t);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += t[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) sh[ps][cq * 4 + e] = acc[e];
  __syncthreads();
  if (tid < 256) {
    const int g = tid >> 5, c = tid & 31;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += sh[g * 16 + i][c];
    sh2[g][c] = s;
  }
  __syncthreads();
  if (tid < 32) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < 8; ++g) s += sh2[g][tid];
    const int64_t oc = (int64_t)blockIdx.x * 32 + tid;
    V *o = a == 0 ? out0 : (a == 1 ? out1 : out2);
    if (oc < cols && o != nullptr) o[oc] = io<V>::to_scalar(s);
  }
}

template <typename V>
static inline int launch_colsum_finalize(const float *part, int64_t P,
                                         int64_t cols, void *out0, void *out1,
                                         hipStream_t st, void *out2 = nullptr,
                                         int narrays = 0) {
  const int64_t grid = ceil_div(cols, 32);
  // narrays = number of arrays of partial rows (outputs that are null are
  // skipped); by default one per non-null output
  if (narrays <= 0) narrays = out1 != nullptr ? 2 : 1;
  colsum_finalize_kernel<V>
      <<<dim3((unsigned)grid, (unsigned)narrays), 1024, 0, st>>>(
          part, P, cols, (V *)out0, (V *)out1, (V *)out2);
  return check_launch("colsum_finalize_kernel");
}

}  // namespace oslo
