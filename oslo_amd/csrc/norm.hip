// LayerNorm / RMSNorm forward and backward for gfx950.
//
// Register-resident path (rows of up to 64 * 16 * 8 chunks): a row is split
// over `wpr` consecutive wavefronts, every lane holds VPL chunks of E
// elements in registers, so x (and dy) are read from HBM exactly once.
// LayerNorm statistics are Welford/Chan: each lane takes the exact mean and
// sum of squared deviations of its own resident elements, the equal-sized
// partials are merged pairwise by a DPP butterfly inside the wave and through
// LDS across the waves of a row (one barrier).  RMSNorm needs one sum.
//
// Backward is a single pass over dy and x: one persistent workgroup per CU
// strides over the rows (the next row is prefetched in packed form), keeps
// the per-column partial sums of dgamma / dbeta in registers for the columns
// its lanes own, and writes one fp32 partial row; a small finalize kernel
// reduces the partial rows in a fixed order (deterministic, no atomics).
//
// Formulas follow oslo/torch/_C/csrc/fused_layer_norm.cu:310-359 (forward)
// and :594-741 (grad input), :458-591 (grad gamma/beta) of the reference.
#include <atomic>
#include <type_traits>

#include "capi.h"
#include "common.hip.h"
#include "colsum.hip.h"

namespace oslo {

// ---------------------------------------------------------------------------
// helpers
// ---------------------------------------------------------------------------
// Sums over the wpr (<= 16) consecutive waves that share a row: lane 0 of every
// wave publishes its wave's sum in LDS, then lane l < wpr of every wave reads
// the sum of wave first + l and one DPP row reduction combines them, which
// costs a fixed dozen instructions instead of a loop over wpr.
// Two simultaneous row sums sharing one barrier.  red is [2][16] floats.
// With LPR < 64 a row belongs to LPR consecutive lanes of one wave (wpr == 1)
// and the sums stay inside that lane group.
template <int LPR = kWave>
__device__ __forceinline__ void row_sum2(float &a, float &b, float *red,
                                         int wave, int first, int wpr,
                                         int lane) {
  if constexpr (LPR < kWave) {
    a = group_allreduce<OpSum, LPR>(a);
    b = group_allreduce<OpSum, LPR>(b);
    return;
  }
  a = wave_sum(a);
  b = wave_sum(b);
  if (wpr > 1) {
    if (lane == 0) {
      red[wave] = a;
      red[16 + wave] = b;
    }
    __syncthreads();
    const bool own = lane < wpr;
    const int src = own ? first + lane : first;
    const float ra = red[src], rb = red[16 + src];
    a = row16_allreduce<OpSum>(own ? ra : 0.f);
    b = row16_allreduce<OpSum>(own ? rb : 0.f);
  }
}

template <int LPR = kWave>
__device__ __forceinline__ float row_sum1(float a, float *red, int wave,
                                          int first, int wpr, int lane) {
  if constexpr (LPR < kWave) return group_allreduce<OpSum, LPR>(a);
  a = wave_sum(a);
  if (wpr > 1) {
    if (lane == 0) red[wave] = a;
    __syncthreads();
    const bool own = lane < wpr;
    const float ra = red[own ? first + lane : first];
    a = row16_allreduce<OpSum>(own ? ra : 0.f);
  }
  return a;
}

// The same sums when a row is a whole number of half-waves ("units" of 32
// lanes, `upr` of them per row; rows of 96 or 160 chunks then leave no lane
// idle): reduction inside the unit, one value per unit through LDS, then every
// lane adds the upr values of its row.  red is [2][32] floats.
__device__ __forceinline__ void unit_sum2(float &a, float &b, float *red,
                                          int unit, int first, int upr,
                                          int ulane) {
  a = group_allreduce<OpSum, 32>(a);
  b = group_allreduce<OpSum, 32>(b);
  if (ulane == 0) {
    red[unit] = a;
    red[32 + unit] = b;
  }
  __syncthreads();
  a = 0.f;
  b = 0.f;
  for (int u = 0; u < upr; ++u) {
    a += red[first + u];
    b += red[32 + first + u];
  }
}

// Welford partials of equal size (every lane holds w.n values) merged over
// the wave and then over the wpr waves of a row.  The waves hold equal
// counts c, so the row's mean is the average of the wave means and its M2 is
// sum_w (M2_w + c (mean_w - mean)^2).  red holds two areas of 48 floats;
// `parity` alternates between them from one call to the next so that a
// single barrier per call suffices.
template <int LPR = kWave>
__device__ __forceinline__ Welford row_welford(Welford w, float *red, int wave,
                                               int first, int wpr, int lane,
                                               int parity) {
  if constexpr (LPR < kWave) {
    // pairwise merges inside the lane group; every merge is symmetric, so
    // the lanes of a group end with the same bits
    float mean = w.mean, m2 = w.m2;
    const float c = w.n;
    merge_equal(mean, m2, dpp_mov<kDppQuadSwap1>(mean), dpp_mov<kDppQuadSwap1>(m2), c);
    merge_equal(mean, m2, dpp_mov<kDppQuadSwap2>(mean), dpp_mov<kDppQuadSwap2>(m2), 2.f * c);
    merge_equal(mean, m2, dpp_mov<kDppRowHalfMirror>(mean), dpp_mov<kDppRowHalfMirror>(m2),
                4.f * c);
    if constexpr (LPR >= 16)
      merge_equal(mean, m2, dpp_mov<kDppRowMirror>(mean), dpp_mov<kDppRowMirror>(m2), 8.f * c);
    if constexpr (LPR >= 32)
      merge_equal(mean, m2, __shfl_xor(mean, 16), __shfl_xor(m2, 16), 16.f * c);
    w.mean = mean;
    w.m2 = m2;
    w.n = c * (float)LPR;
    return w;
  }
  w = wave_welford_equal(w.mean, w.m2, w.n);
  if (wpr > 1) {
    float *area = red + parity * 48;
    if (lane == 0) {
      area[wave] = w.mean;
      area[16 + wave] = w.m2;
    }
    __syncthreads();
    const bool own = lane < wpr;
    const int src = own ? first + lane : first;
    const float mw = area[src], qw = area[16 + src];
    const float mean =
        row16_allreduce<OpSum>(own ? mw : 0.f) * __builtin_amdgcn_rcpf((float)wpr);
    const float d = mw - mean;
    const float m2 = row16_allreduce<OpSum>(own ? fmaf(w.n * d, d, qw) : 0.f);
    w.mean = mean;
    w.m2 = m2;
    w.n *= (float)wpr;
  }
  return w;
}

// ---------------------------------------------------------------------------
// forward, register-resident
// ---------------------------------------------------------------------------
// Operands of the fused prologue h = dropout(x + bias) + residual, which the
// FUSE build of the forward kernel evaluates, rounds to the storage type and
// (optionally) stores before it normalises h: the chain FusedBiasDropout ->
// residual add -> LayerNorm of oslo/transformers/models/bert/modeling_bert.py:
// 343-346, 446-449 in one pass.  One dtype for all tensors.
struct FusePrologue {
  const void *bias;      // [n2] or null
  const void *residual;  // [n1, n2] or null
  void *h_out;           // [n1, n2] or null
  DropArgs d;
  int drop;              // 1: dropout with d, 0: none
};

// EVEN: every lane holds exactly VPL chunks of its row (no column guards;
// LayerNorm then merges equal-sized Welford partials).
// LPR: lanes that hold a row.  64: a row takes wpr whole waves.  8, 16, 32:
// rows of at most LPR chunks lie side by side in a wave (VPL == 1, wpr == 1,
// and rpb counts the rows of all lane groups of the workgroup); rows of
// exactly 3 * LPR chunks (768 16-bit elements = 96 chunks = 32 lanes x 3)
// take VPL == 3.
template <typename T, typename V, int VPL, bool RMS, bool EVEN, int MAXT,
          bool FUSE = false, int LPR = kWave>
__global__ __launch_bounds__(MAXT) void norm_fwd_reg_kernel(
    const T *__restrict__ x, const V *__restrict__ gamma,
    const V *__restrict__ beta, V *__restrict__ y, float *__restrict__ mean,
    float *__restrict__ invvar, int64_t n1, int n2, float eps, int wpr,
    int rpb, int iters, FusePrologue fp) {
  constexpr int E = chunk_elems<T, V>::value;
  static_assert(!FUSE || sizeof(T) == sizeof(V), "fused prologue: one dtype");
  if constexpr (FUSE) fp.d = resolve_drop(fp.d);
  static_assert(LPR == kWave || VPL == 1 || VPL == 3, "side-by-side rows: one or three chunks per lane");
  __shared__ float red[2][48];
  const int lane = threadIdx.x & 63;
  // the wave index is uniform: keep it (and the row arithmetic) in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int SUB = kWave / LPR;
  const int first = (wave / wpr) * wpr;
  const int rslot = LPR == kWave ? wave / wpr : wave * SUB + lane / LPR;
  const int nchunks = n2 / E;
  const int cstride = LPR == kWave ? kWave * wpr : LPR;
  const int c0 = LPR == kWave ? (wave - first) * kWave + lane : (lane & (LPR - 1));
  const float fn = (float)n2;
  int parity = 0;

  // the affine parameters of this lane's columns stay packed in registers
  // for all rows of the workgroup
  RawChunk<V, E> graw[VPL], braw[VPL];
  if (gamma != nullptr) {
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (c < nchunks) {
        graw[k].load_cached(gamma + (int64_t)c * E);
        if constexpr (!RMS) braw[k].load_cached(beta + (int64_t)c * E);
      }
    }
  }

  const T *fbias = static_cast<const T *>(fp.bias);
  const T *fres = static_cast<const T *>(fp.residual);
  T *fh = static_cast<T *>(fp.h_out);
  RawChunk<T, E> biasraw[FUSE ? VPL : 1];
  if constexpr (FUSE) {
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (fbias != nullptr && c < nchunks)
        biasraw[k].load_cached(fbias + (int64_t)c * E);
      else
        biasraw[k].zero();
    }
  }

  // A workgroup takes `iters` consecutive groups of rpb rows, then strides
  // by the grid.
  const int64_t total_groups = (n1 + rpb - 1) / rpb;
  // The next row of a workgroup is requested, in packed form, before the
  // current one is reduced, so that every wave keeps loads in flight.
  // (not in the 1024-thread build with 32 elements per lane, whose register
  // budget of 128 has no room for the second row)
  constexpr bool kPrefetch = !(MAXT > 256 && VPL * E >= 32);
  RawChunk<T, E> nx[VPL];
  RawChunk<T, E> nr[FUSE ? VPL : 1];  // residual of the fused prologue
  auto fetch = [&](int64_t group) {
    int64_t frow = group * rpb + rslot;
    // a slot past the last row re-reads row n1 - 1 and stores nothing
    frow = frow < n1 ? frow : n1 - 1;
    const T *xr = x + frow * n2;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (EVEN || c < nchunks)
        nx[k].load(xr + (int64_t)c * E);
      else
        nx[k].zero();
      if constexpr (FUSE) {
        if (fres != nullptr && (EVEN || c < nchunks))
          nr[k].load(fres + frow * n2 + (int64_t)c * E);
        else
          nr[k].zero();
      }
    }
  };
  for (int64_t g0 = (int64_t)blockIdx.x * iters; g0 < total_groups;
       g0 += (int64_t)gridDim.x * iters) {
  if constexpr (kPrefetch) fetch(g0);
  for (int it = 0; it < iters && g0 + it < total_groups; ++it) {
    const int64_t row = (g0 + it) * rpb + rslot;
    const bool rvalid = row < n1;
    float v[VPL][E];
    if constexpr (!kPrefetch) fetch(g0 + it);
#pragma unroll
    for (int k = 0; k < VPL; ++k) nx[k].unpack(v[k]);
    if constexpr (FUSE) {
      // h = dropout(x + bias) + residual, rounded once to the storage type;
      // the statistics below are those of the stored h.  Done before the
      // next row is requested, so the packed residual is dead by then.
#pragma unroll
      for (int k = 0; k < VPL; ++k) {
        const int c = c0 + k * cstride;
        if (EVEN || c < nchunks) {
          float b[E], res[E];
          biasraw[k].unpack(b);
          nr[k].unpack(res);
          uint32_t keep = (1u << E) - 1u;
          if (fp.drop) keep = chunk_keep_bits<E>(rvalid ? row : n1 - 1, n2, c, fp.d);
#pragma unroll
          for (int e = 0; e < E; ++e) {
            float t = v[k][e] + b[e];
            if (fp.drop) t = (keep >> e) & 1u ? t * fp.d.scale : 0.f;
            v[k][e] = io<T>::round(t + res[e]);
          }
          if (fh != nullptr && rvalid)
            store_chunk<T, E>(fh + row * n2 + (int64_t)c * E, v[k]);
        }
      }
    }
    if constexpr (kPrefetch) {
      if (it + 1 < iters && g0 + it + 1 < total_groups) fetch(g0 + it + 1);
    }

    float mu = 0.f, q = 0.f;
    if constexpr (!RMS && EVEN) {
      // Welford / Chan: exact mean and sum of squared deviations of the
      // lane's own (register-resident) elements, then pairwise merges of the
      // equal-sized (mean, M2) partials across lanes and waves: one barrier.
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < VPL; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) s += v[k][e];
      Welford w;
      w.n = (float)(VPL * E);
      w.mean = s * (1.0f / (float)(VPL * E));
      w.m2 = 0.f;
#pragma unroll
      for (int k = 0; k < VPL; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const float d = v[k][e] - w.mean;
          w.m2 += d * d;
        }
      w = row_welford<LPR>(w, &red[0][0], wave, first, wpr, lane, parity);
      parity ^= 1;
      mu = w.mean;
      q = w.m2;
    } else if constexpr (!RMS) {
      // ragged rows: the two-pass form, mean first, then the squared
      // deviations of the valid elements
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < VPL; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) s += v[k][e];
      s = row_sum1<LPR>(s, &red[0][0], wave, first, wpr, lane);
      mu = s / fn;
#pragma unroll
      for (int k = 0; k < VPL; ++k) {
        if (c0 + k * cstride < nchunks) {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            const float d = v[k][e] - mu;
            q += d * d;
          }
        }
      }
      q = row_sum1<LPR>(q, &red[1][0], wave, first, wpr, lane);
    } else {
#pragma unroll
      for (int k = 0; k < VPL; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) q += v[k][e] * v[k][e];
      q = row_sum1<LPR>(q, red[parity], wave, first, wpr, lane);
      parity ^= 1;
    }
    const float rs = rsqrt_refined(q / fn + eps);

    if (rvalid) {
      V *yr = y + row * n2;
#pragma unroll
      for (int k = 0; k < VPL; ++k) {
        const int c = c0 + k * cstride;
        if (c < nchunks) {
          float o[E];
          if constexpr (!RMS) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = (v[k][e] - mu) * rs;
            if (gamma != nullptr) {
              float g[E], b[E];
              graw[k].unpack(g);
              braw[k].unpack(b);
#pragma unroll
              for (int e = 0; e < E; ++e) o[e] = o[e] * g[e] + b[e];
            }
          } else {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = io<V>::round(v[k][e] * rs);
            if (gamma != nullptr) {
              float g[E];
              graw[k].unpack(g);
#pragma unroll
              for (int e = 0; e < E; ++e) o[e] = g[e] * o[e];
            }
          }
          store_chunk<V, E>(yr + (int64_t)c * E, o);
        }
      }
      if (c0 == 0) {
        if constexpr (!RMS) mean[row] = mu;
        invvar[row] = rs;
      }
    }
  }
  }
}

// ---------------------------------------------------------------------------
// forward, generic (any n2, any alignment): one 256-thread workgroup per row,
// streaming Welford per thread merged with Chan's formula; second pass
// re-reads the row (L2-resident).
// ---------------------------------------------------------------------------
template <typename T, typename V, bool RMS>
__global__ __launch_bounds__(256) void norm_fwd_generic_kernel(
    const T *__restrict__ x, const V *__restrict__ gamma,
    const V *__restrict__ beta, V *__restrict__ y, float *__restrict__ mean,
    float *__restrict__ invvar, int64_t n1, int64_t n2, float eps) {
  __shared__ float sh[3][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int64_t row = blockIdx.x; row < n1; row += gridDim.x) {
    const T *xr = x + row * n2;
    Welford w{0.f, 0.f, 0.f};
    for (int64_t i = tid; i < n2; i += 256) {
      const float v = io<T>::from_scalar(xr[i]);
      if constexpr (RMS) {
        w.m2 += v * v;
      } else {
        // Welford's online update (fused_layer_norm.cu:12-19 of the reference)
        w.n += 1.f;
        const float d = v - w.mean;
        w.mean += d / w.n;
        w.m2 += d * (v - w.mean);
      }
    }
    if constexpr (RMS)
      w.m2 = wave_sum(w.m2);
    else
      w = wave_welford(w);
    if (lane == 0) {
      sh[0][wave] = w.n;
      sh[1][wave] = w.mean;
      sh[2][wave] = w.m2;
    }
    __syncthreads();
    Welford t{sh[0][0], sh[1][0], sh[2][0]};
    for (int k = 1; k < 4; ++k) {
      const Welford o{sh[0][k], sh[1][k], sh[2][k]};
      if constexpr (RMS)
        t.m2 += o.m2;
      else
        t = chan_merge(t, o);
    }
    __syncthreads();
    const float mu = RMS ? 0.f : t.mean;
    const float rs = 1.0f / sqrtf(t.m2 / (float)n2 + eps);
    V *yr = y + row * n2;
    for (int64_t i = tid; i < n2; i += 256) {
      const float v = io<T>::from_scalar(xr[i]);
      float o;
      if constexpr (!RMS) {
        o = (v - mu) * rs;
        if (gamma != nullptr)
          o = o * io<V>::from_scalar(gamma[i]) + io<V>::from_scalar(beta[i]);
      } else {
        o = io<V>::round(v * rs);
        if (gamma != nullptr) o = io<V>::from_scalar(gamma[i]) * o;
      }
      yr[i] = io<V>::to_scalar(o);
    }
    if (tid == 0) {
      if constexpr (!RMS) mean[row] = mu;
      invvar[row] = rs;
    }
  }
}

// ---------------------------------------------------------------------------
// backward, register-resident, single pass
// ---------------------------------------------------------------------------
// EVEN: every lane holds exactly VPL chunks of its row (no column guards).
// Operands of the fused epilogue, the backward of the forward kernel's
// prologue h = dropout(x + bias) + residual: the gradient of h is the norm's
// input gradient plus dh_extra (what reaches h from its other consumers); it
// is stored through the kernel's dx pointer (= gradient of the residual) and,
// masked and scaled, through dx_drop (= gradient of x); the column sums of
// dx_drop as stored are the bias gradient (an extra array of partial rows).
struct FuseEpilogue {
  const void *dh_extra;  // [n1, n2] or null
  void *dx_drop;         // [n1, n2] or null
  DropArgs d;
  int drop;              // 1: dropout with d, 0: none
  int want_dbias;        // 1: partial rows of the bias gradient are written
};

// MAXT: largest workgroup the build is launched with (768 leaves a third more
// registers per lane than 1024, which the 16-elements-per-lane builds need).
// LPR: as in the forward kernel (rows side by side in a wave when < 64).
// UNIT: 64, or 32 when a row is `wpr` half-waves (then "wave" below means
// such a unit of 32 lanes; LPR == 64, VPL == 1, EVEN).
template <typename T, typename V, int VPL, bool RMS, bool EVEN, int PF,
          bool FUSE = false, int MAXT = 1024, int LPR = kWave, int UNIT = kWave>
__global__ __launch_bounds__(MAXT) void norm_bwd_reg_kernel(
    const V *__restrict__ dy, const T *__restrict__ x,
    const float *__restrict__ mean, const float *__restrict__ invvar,
    const V *__restrict__ gamma, T *__restrict__ dx, float *__restrict__ part,
    int64_t n1, int n2, int wpr, int rpb, FuseEpilogue fe) {
  constexpr int E = chunk_elems<T, V>::value;
  static_assert(!FUSE || sizeof(T) == sizeof(V), "fused epilogue: one dtype");
  if constexpr (FUSE) fe.d = resolve_drop(fe.d);
  static_assert(LPR == kWave || VPL == 1 || VPL == 3, "side-by-side rows: one or three chunks per lane");
  static_assert(UNIT == kWave || (UNIT == 32 && LPR == kWave && VPL == 1 && EVEN),
                "half-wave units: whole-unit rows, one chunk per lane");
  extern __shared__ __align__(16) float xslot[];  // [n2] when rpb > 1
  __shared__ float red[2][64];
  const int lane = UNIT == kWave ? (threadIdx.x & 63) : (threadIdx.x & 31);
  // the wave index is uniform: keep it (and the row arithmetic) in scalar registers
  const int wave = UNIT == kWave ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6)
                                 : (int)(threadIdx.x >> 5);
  constexpr int SUB = kWave / LPR;
  const int first = (wave / wpr) * wpr;
  // row slot of this lane; wslot is the wave's slot when its lane groups
  // have been folded into one
  const int wslot = wave / wpr;
  const int rslot = LPR == kWave ? wslot : wave * SUB + lane / LPR;
  const int nchunks = n2 / E;
  const int cstride = LPR == kWave ? UNIT * wpr : LPR;
  const int c0 = LPR == kWave ? (wave - first) * UNIT + lane : (lane & (LPR - 1));
  const float fn = (float)n2;
  const bool affine = gamma != nullptr;

  // gamma stays packed (half the registers) and is unpacked once per row.
  // With 16 elements per lane the registers run out: all but GREG chunks of
  // gamma then live in LDS, each lane reading back what it wrote (no barrier).
  constexpr int GREG = VPL * E >= 16 ? (sizeof(V) == 4 ? 1 : 0) : VPL;
  RawChunk<V, E> gmraw[GREG > 0 ? GREG : 1];
  RawChunk<V, E> *const gslot =
      reinterpret_cast<RawChunk<V, E> *>(xslot + (rpb > SUB ? n2 : 0));
  float acc_g[VPL][E], acc_b[VPL][E];
  float acc_d[FUSE ? VPL : 1][E];  // bias gradient of the fused epilogue
#pragma unroll
  for (int k = 0; k < VPL; ++k) {
    const int c = c0 + k * cstride;
    RawChunk<V, E> g;
    if (affine && c < nchunks)
      g.load_cached(gamma + (int64_t)c * E);
    else
      g.zero();
    if constexpr (GREG == VPL) {
      gmraw[k] = g;
    } else {
      if (k < GREG)
        gmraw[k < GREG ? k : 0] = g;
      else
        gslot[(k - GREG) * blockDim.x + threadIdx.x] = g;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
      acc_g[k][e] = 0.f;
      acc_b[k][e] = 0.f;
      if constexpr (FUSE) acc_d[k][e] = 0.f;
    }
  }
  const T *fextra = static_cast<const T *>(fe.dh_extra);
  T *fdrop = static_cast<T *>(fe.dx_drop);

  // The loads of a row are issued PF iterations ahead, in packed form, so
  // that they are in flight while the previous rows are reduced and stored.
  struct RowFetch {
    RawChunk<V, E> d[VPL];
    RawChunk<T, E> x[VPL];
    RawChunk<T, E> extra[FUSE ? VPL : 1];
    float mu, rs;
  };
  const int64_t rstride = (int64_t)gridDim.x * rpb;
  // A slot past the last row re-reads row n1 - 1 (its results are discarded),
  // which keeps the loads unconditional.
  auto fetch = [&](RowFetch &f, int64_t base) {
    int64_t frow = base + rslot;
    frow = frow < n1 ? frow : n1 - 1;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (EVEN || c < nchunks) {
        f.d[k].load(dy + frow * n2 + (int64_t)c * E);
        f.x[k].load(x + frow * n2 + (int64_t)c * E);
      } else {
        f.d[k].zero();
        f.x[k].zero();
      }
      if constexpr (FUSE) {
        if (fextra != nullptr && (EVEN || c < nchunks))
          f.extra[k].load(fextra + frow * n2 + (int64_t)c * E);
        else
          f.extra[k].zero();
      }
    }
    f.mu = RMS ? 0.f : mean[frow];
    f.rs = invvar[frow];
  };

  int parity = 0;
  // One row per slot: consume the fetched row, refill the buffer with the row
  // PF iterations later, reduce, store dx.
  auto process = [&](RowFetch &f, int64_t base) {
    const int64_t row = base + rslot;
    const bool rvalid = row < n1;
    float d[VPL][E], xh[VPL][E];
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      f.d[k].unpack(d[k]);
      f.x[k].unpack(xh[k]);
    }
    if (!rvalid) {  // wave-uniform: a slot past the end contributes nothing
#pragma unroll
      for (int k = 0; k < VPL; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) d[k][e] = 0.f;
    }
    const float mu = f.mu, rs = f.rs;
    float extra[FUSE ? VPL : 1][E];
    if constexpr (FUSE) {
#pragma unroll
      for (int k = 0; k < VPL; ++k) f.extra[k].unpack(extra[k]);
    }
    fetch(f, base + PF * rstride);
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      float gm[E];
      if (k < GREG)
        gmraw[k < GREG ? k : 0].unpack(gm);
      else
        gslot[(k - GREG) * blockDim.x + threadIdx.x].unpack(gm);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        // normalised input; subtract first: exact when x is close to the mean
        const float h = (xh[k][e] - mu) * rs;
        const float dg = affine ? d[k][e] * gm[e] : d[k][e];
        xh[k][e] = h;
        s1 += dg;
        s2 += dg * h;
        acc_g[k][e] += d[k][e] * h;
        acc_b[k][e] += d[k][e];
        d[k][e] = dg;  // only dy * gamma is needed from here on
      }
    }
    if constexpr (UNIT == 32) {
      unit_sum2(s1, s2, red[parity], wave, first, wpr, lane);
      if constexpr (RMS) s1 = 0.f;
    } else if constexpr (RMS) {
      s2 = row_sum1<LPR>(s2, red[parity], wave, first, wpr, lane);
      s1 = 0.f;
    } else {
      row_sum2<LPR>(s1, s2, red[parity], wave, first, wpr, lane);
    }
    parity ^= 1;
    // dx = invvar / n2 * (n2 * dy * gamma - s1 - xhat * s2), regrouped as
    // invvar * (dy * gamma) - b1 - c2 * xhat
    const float term = rs / fn;
    const float b1 = term * s1, c2 = term * s2;
    if (rvalid) {
      T *dxr = dx + row * n2;
#pragma unroll
      for (int k = 0; k < VPL; ++k) {
        const int c = c0 + k * cstride;
        if (EVEN || c < nchunks) {
          float o[E];
#pragma unroll
          for (int e = 0; e < E; ++e)
            o[e] = fmaf(-c2, xh[k][e], fmaf(rs, d[k][e], -b1));
          if constexpr (FUSE) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] += extra[k][e];
          }
          if constexpr (!FUSE) {
            store_chunk<T, E>(dxr + (int64_t)c * E, o);
          } else if (fe.drop) {
            // gradient of x of the prologue: masked and scaled from the
            // unrounded gradient of h, then rounded once
            store_chunk<T, E>(dxr + (int64_t)c * E, o);
            const uint32_t keep = chunk_keep_bits<E>(row, n2, c, fe.d);
#pragma unroll
            for (int e = 0; e < E; ++e)
              o[e] = (keep >> e) & 1u ? o[e] * fe.d.scale : 0.f;
            store_chunk_readback<T, E>(
                fdrop != nullptr ? fdrop + row * n2 + (int64_t)c * E : nullptr, o);
#pragma unroll
            for (int e = 0; e < E; ++e) acc_d[k][e] += o[e];  // dx as stored
          } else {
            // no dropout: the gradient of x is the gradient of h as stored
            store_chunk_readback<T, E>(dxr + (int64_t)c * E, o);
            if (fdrop != nullptr)
              store_chunk<T, E>(fdrop + row * n2 + (int64_t)c * E, o);
#pragma unroll
            for (int e = 0; e < E; ++e) acc_d[k][e] += o[e];
          }
        }
      }
    }
  };

  const int64_t base0 = (int64_t)blockIdx.x * rpb;
  if constexpr (PF == 1) {
    RowFetch f0;
    fetch(f0, base0);
    for (int64_t base = base0; base < n1; base += rstride) process(f0, base);
  } else {
    RowFetch f0, f1;
    fetch(f0, base0);
    fetch(f1, base0 + rstride);
    for (int64_t base = base0; base < n1; base += 2 * rstride) {
      process(f0, base);
      if (base + rstride >= n1) break;  // uniform over the workgroup
      process(f1, base + rstride);
    }
  }

  if (part == nullptr) return;  // uniform: no parameter gradients wanted

  // Fold the row slots of this workgroup into slot 0, one slot at a time.
  // Arrays: 0 = dgamma, then dbeta (LayerNorm only), then the bias gradient of
  // the fused epilogue (last, when wanted).
  constexpr int NARR = RMS ? 1 : 2;
  const int64_t P = gridDim.x;
  // (a lambda over one accumulator array at a time keeps the arrays in
  // registers: none of them is indexed by a run-time value)
  const int wslots = LPR == kWave ? rpb : rpb / SUB;  // wave-level row slots
  const bool lead = LPR == kWave || lane < LPR;        // first lane group
  auto fold_and_store = [&](auto &acc, int a) {
    if constexpr (LPR < kWave) {
      // the lane groups of a wave hold the same columns: sum them into the
      // first group
#pragma unroll
      for (int k = 0; k < VPL; ++k)
#pragma unroll
        for (int e = 0; e < E; ++e) {
          float t = acc[k][e];
#pragma unroll
          for (int o = LPR; o < kWave; o <<= 1) t += __shfl_xor(t, o);
          acc[k][e] = t;
        }
    }
    for (int s = 1; s < wslots; ++s) {
      __syncthreads();
      if (wslot == s && lead) {
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
          const int c = c0 + k * cstride;
          if (c < nchunks) {
#pragma unroll
            for (int e = 0; e < E; ++e) xslot[c * E + e] = acc[k][e];
          }
        }
      }
      __syncthreads();
      if (wslot == 0 && lead) {
#pragma unroll
        for (int k = 0; k < VPL; ++k) {
          const int c = c0 + k * cstride;
          if (c < nchunks) {
#pragma unroll
            for (int e = 0; e < E; ++e) acc[k][e] += xslot[c * E + e];
          }
        }
      }
    }
    if (wslot == 0 && lead) {
      float *prow = part + ((int64_t)a * P + blockIdx.x) * n2;
#pragma unroll
      for (int k = 0; k < VPL; ++k) {
        const int c = c0 + k * cstride;
        if (c < nchunks) store_chunk<float, E>(prow + (int64_t)c * E, acc[k]);
      }
    }
  };
  fold_and_store(acc_g, 0);
  if constexpr (!RMS) fold_and_store(acc_b, 1);
  if constexpr (FUSE) {
    if (fe.want_dbias) fold_and_store(acc_d, NARR);
  }
}

// ---------------------------------------------------------------------------
// backward, generic: dx per row by one workgroup (two passes over the row),
// parameter gradients by one thread per column walking all rows.
// ---------------------------------------------------------------------------
template <typename T, typename V, bool RMS>
__global__ __launch_bounds__(256) void norm_bwd_dx_generic_kernel(
    const V *__restrict__ dy, const T *__restrict__ x,
    const float *__restrict__ mean, const float *__restrict__ invvar,
    const V *__restrict__ gamma, T *__restrict__ dx, int64_t n1, int64_t n2,
    FuseEpilogue fe) {
  // fe: the fused epilogue (all-null for the plain backward): dh_extra is added
  // before the single rounding, dx_drop receives the masked, scaled gradient
  fe.d = resolve_drop(fe.d);
  const T *extra = static_cast<const T *>(fe.dh_extra);
  T *dx_drop = static_cast<T *>(fe.dx_drop);
  __shared__ float sh[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int64_t row = blockIdx.x; row < n1; row += gridDim.x) {
    const V *dyr = dy + row * n2;
    const T *xr = x + row * n2;
    const float mu = RMS ? 0.f : mean[row];
    const float rs = invvar[row];
    float s1 = 0.f, s2 = 0.f;
    for (int64_t i = tid; i < n2; i += 256) {
      const float g = gamma ? io<V>::from_scalar(gamma[i]) : 1.f;
      const float dg = io<V>::from_scalar(dyr[i]) * g;
      const float h = (io<T>::from_scalar(xr[i]) - mu) * rs;
      s1 += dg;
      s2 += dg * h;
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    if (lane == 0) {
      sh[0][wave] = s1;
      sh[1][wave] = s2;
    }
    __syncthreads();
    s1 = (sh[0][0] + sh[0][1]) + (sh[0][2] + sh[0][3]);
    s2 = (sh[1][0] + sh[1][1]) + (sh[1][2] + sh[1][3]);
    __syncthreads();
    if constexpr (RMS) s1 = 0.f;
    const float fn = (float)n2;
    const float term = rs / fn;
    T *dxr = dx + row * n2;
    for (int64_t i = tid; i < n2; i += 256) {
      const float g = gamma ? io<V>::from_scalar(gamma[i]) : 1.f;
      const float h = (io<T>::from_scalar(xr[i]) - mu) * rs;
      float f = fn * io<V>::from_scalar(dyr[i]) * g;
      f -= s1;
      f -= h * s2;
      float o = f * term;
      if (extra != nullptr) o += io<T>::from_scalar(extra[row * n2 + i]);
      dxr[i] = io<T>::to_scalar(o);
      if (dx_drop != nullptr) {
        if (fe.drop) o = keep_element(row * n2 + i, fe.d) ? o * fe.d.scale : 0.f;
        dx_drop[row * n2 + i] = io<T>::to_scalar(o);
      }
    }
  }
}

template <typename T, typename V, bool RMS>
__global__ __launch_bounds__(256) void norm_bwd_param_generic_kernel(
    const V *__restrict__ dy, const T *__restrict__ x,
    const float *__restrict__ mean, const float *__restrict__ invvar,
    V *__restrict__ dgamma, V *__restrict__ dbeta, int64_t n1, int64_t n2) {
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= n2) return;
  float ag = 0.f, ab = 0.f;
  for (int64_t row = 0; row < n1; ++row) {
    const float mu = RMS ? 0.f : mean[row];
    const float d = io<V>::from_scalar(dy[row * n2 + col]);
    ag += d * (io<T>::from_scalar(x[row * n2 + col]) - mu) * invvar[row];
    ab += d;
  }
  dgamma[col] = io<V>::to_scalar(ag);
  if constexpr (!RMS) dbeta[col] = io<V>::to_scalar(ab);
}

// Functor of the generic column sums: dgamma (and dbeta) contributions.
template <typename T, typename V, bool RMS> struct NormParamGrad {
  const V *dy;
  const T *x;
  const float *mean;
  const float *invvar;
  int64_t n2;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float *acc) const {
    const float mu = RMS ? 0.f : mean[r];
    const float d = io<V>::from_scalar(dy[r * n2 + c]);
    acc[0] += d * (io<T>::from_scalar(x[r * n2 + c]) - mu) * invvar[r];
    if constexpr (!RMS) acc[1] += d;
  }
};

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct RowSplit {
  int vpl;  // chunks per lane (template value)
  int wpr;  // waves per row
  int rpb;  // rows per workgroup iteration
  bool ok;
};

// Splits a row of `nchunks` chunks over waves so that a lane holds at most
// `cap` chunks; `allowed` lists the instantiated VPL values (ascending).
static RowSplit split_row(int64_t nchunks, int cap, const int *allowed,
                          int nallowed, int min_waves) {
  RowSplit r{0, 1, 1, false};
  if (nchunks <= 0) return r;
  int64_t wpr = ceil_div(nchunks, (int64_t)kWave * cap);
  if (wpr > 16) return r;
  int64_t vpl = ceil_div(nchunks, kWave * wpr);
  for (int i = 0; i < nallowed; ++i) {
    if (allowed[i] >= vpl) {
      r.vpl = allowed[i];
      r.wpr = (int)wpr;
      int rpb = min_waves / r.wpr;
      if (rpb < 1) rpb = 1;
      while (rpb * r.wpr > 16) --rpb;
      r.rpb = rpb;
      r.ok = true;
      return r;
    }
  }
  return r;
}

// Lanes that hold a row of `nchunks` chunks: 64, or 8 / 16 / 32 when the row
// is short enough for several rows to lie side by side in a wave.
static int lanes_per_row(int64_t nchunks) {
  if (nchunks > 32 || g_tune.norm_lanes_per_row == kWave) return kWave;
  int lpr = nchunks <= 8 ? 8 : nchunks <= 16 ? 16 : 32;
  const int t = g_tune.norm_lanes_per_row;
  if ((t == 8 || t == 16 || t == 32) && t >= lpr) lpr = t;
  return lpr;
}

// Rows of exactly 3 * 8, 3 * 16 or 3 * 32 chunks (hidden sizes 192, 384, 768
// in a 16-bit type): lanes per row for the three-chunks-per-lane builds, else 0.
static int lanes_per_row_x3(int64_t nchunks) {
  if (g_tune.norm_lanes_per_row == kWave || nchunks % 3 != 0) return 0;
  const int64_t q = nchunks / 3;
  return q == 8 || q == 16 || q == 32 ? (int)q : 0;
}

int64_t colsum_parts_norm(int64_t n1, int64_t n2) {
  (void)n2;
  int bpc = g_tune.norm_bwd_blocks_per_cu > 0 ? g_tune.norm_bwd_blocks_per_cu : 1;
  int64_t p = (int64_t)device_cu_count() * bpc;
  if (p > n1) p = n1;
  if (p < 1) p = 1;
  return p;
}

constexpr int kNotFused = 1;  // launch_norm_fwd: shape needs the composed path

// fp != nullptr selects the fused prologue (T == V); shapes outside the
// register path then return kNotFused without launching anything.
template <typename T, typename V, bool RMS>
static int launch_norm_fwd(const void *x, const void *gamma, const void *beta,
                           void *y, float *mean, float *invvar, int64_t n1,
                           int64_t n2, float eps, hipStream_t st,
                           const FusePrologue *fp = nullptr) {
  constexpr int E = chunk_elems<T, V>::value;
  constexpr bool kCanFuse = sizeof(T) == sizeof(V);
  const bool fused = fp != nullptr;
  const bool vec_ok = n2 % E == 0 && aligned16(x) && aligned16(y) &&
                      aligned16(gamma) && aligned16(beta) &&
                      (!fused || (aligned16(fp->bias) && aligned16(fp->residual) &&
                                  aligned16(fp->h_out))) &&
                      n2 <= (int64_t)kWave * 16 * 8 * E;
  static const int kVpl[] = {1, 2, 4, 8};
  RowSplit sp{0, 1, 1, false};
  if (vec_ok) {
    // measured fastest on MI355X: up to four chunks per lane; LayerNorm,
    // whose kernel holds more live registers, takes two in rows of up to four
    // waves that four per lane would not fill evenly (3072 16-bit elements:
    // three waves of two chunks rather than two waves of three), and so do
    // rows of 1536 eight-element chunks (12288 elements: twelve waves measure
    // 5 % faster than six)
    const int64_t nch = n2 / E;
    int cap = (!RMS && nch <= kWave * 2 * 4 && nch % (kWave * 4) != 0) ? 2 : 4;
    if (E == 8 && nch == 1536) cap = 2;
    // rows of 8200 ... 12288 16-bit elements: two chunks per lane over up to
    // twelve waves measure 5-13 % faster than four over five or six
    // (LayerNorm bf16 [8192, 9216] 67 -> 58 us, [8192, 11264] 70 -> 66 us);
    // RMSNorm gains up to 16384 elements together with two row groups per
    // workgroup (below): [8192, 11264] 68 -> 61 us, [8192, 15360] 86 -> 84.5 us
    if (E == 8 && nch > kWave * 4 * 4 && (RMS || nch <= kWave * 2 * 12)) cap = 2;
    // fp32 rows of 3072 and 4096 elements: 3 % faster over twice the waves
    if (E == 4 && (nch == 768 || nch == 1024)) cap = 2;
    // fp16 LayerNorm: four chunks per lane spill in the builds for more than
    // four waves (128 VGPRs), 20 % slower at 10240 elements than two per lane
    // (beyond twelve waves of two the four-chunk build wins again: 13312
    //  elements 95 -> 80 us, 15360 elements 101 -> 89 us)
    if (!RMS && std::is_same<T, _Float16>::value && nch > kWave * 4 * 4 && nch <= kWave * 2 * 12)
      cap = 2;
    // LayerNorm rows of 768 eight-element chunks (6144 elements): four waves of
    // three chunks measure 1.3 % faster than three waves of four (35.7 against
    // 36.1 us for [8192, 6144]); RMSNorm shows no gain
    if (!RMS && E == 8 && nch == 768) cap = 3;
    if (g_tune.norm_fwd_vpl > 0) cap = g_tune.norm_fwd_vpl;
    const int waves = g_tune.norm_fwd_waves > 0 ? g_tune.norm_fwd_waves : 4;
    static const int kVpl3[] = {1, 2, 3, 4, 8};
    if (cap == 3 && !RMS)
      sp = split_row(n2 / E, 3, kVpl3, 5, waves);
    else
      sp = split_row(n2 / E, cap > 8 ? 8 : cap, kVpl, 4, waves);
    // more than 32 resident elements per lane only fit the register budget
    // of a workgroup of at most 256 threads
    if (sp.ok && sp.wpr * sp.rpb > 4 && sp.vpl * E > 32)
      sp = split_row(n2 / E, 32 / E, kVpl, 4, waves);
  }
  // The fused build holds two more packed operands per chunk: at most 16
  // elements per lane.  Measured on MI355X: 16 per lane while a row then fits
  // four waves, else 8 per lane over up to twelve waves, else 16 per lane.
  bool fused_big = false;
  if (fused && vec_ok) {
    const int waves = g_tune.norm_fwd_waves > 0 ? g_tune.norm_fwd_waves : 4;
    if (g_tune.norm_fwd_vpl > 0) {
      const int cap = g_tune.norm_fwd_vpl < 16 / E ? g_tune.norm_fwd_vpl : 16 / E;
      sp = split_row(n2 / E, cap, kVpl, 4, waves);
    } else {
      sp = split_row(n2 / E, 16 / E, kVpl, 4, waves);
      if (!sp.ok || sp.wpr > 4) {
        // (8 per lane measures 20 % slower once it needs 14 or more waves:
        //  rows of 7168 and 8192 16-bit elements)
        const RowSplit narrow = split_row(n2 / E, 8 / E, kVpl, 4, waves);
        if (sp.ok && sp.wpr == 5)
          // rows of 5120 16-bit elements: three rows of five waves per
          // workgroup measure 8 % faster than ten waves at 8 per lane
          sp = split_row(n2 / E, 16 / E, kVpl, 4, 16);
        else if (narrow.ok && (!sp.ok || narrow.wpr <= 12))
          sp = narrow;
      }
    }
    if (sp.ok && sp.vpl * E > 16) sp.ok = false;
    fused_big = sp.ok && sp.wpr * sp.rpb > 4;
  }
  if (fused && !sp.ok) return kNotFused;
  if (!sp.ok) {
    int64_t grid = n1 < 65535 * 16 ? n1 : 65535 * 16;
    norm_fwd_generic_kernel<T, V, RMS><<<dim3((unsigned)grid), 256, 0, st>>>(
        (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean, invvar,
        n1, n2, eps);
    return check_launch("norm_fwd_generic_kernel");
  }
  const int threads = kWave * sp.wpr * sp.rpb;
  // every lane holds exactly vpl chunks: LayerNorm takes the Welford path
  const bool even = (n2 / E) == (int64_t)sp.vpl * kWave * sp.wpr;
  // rows per workgroup = rpb * iters: the workgroup's loads of gamma and beta
  // are spread over that many rows
  // (LayerNorm: two groups, the second one prefetched; RMSNorm is fastest
  // with short-lived workgroups)
  int iters = g_tune.norm_fwd_iters > 0 ? g_tune.norm_fwd_iters
              : (RMS && !(E == 8 && n2 / E > kWave * 4 * 4)) ? 1 : 2;
  int64_t grid = ceil_div(ceil_div(n1, sp.rpb), iters);
  const int64_t maxgrid = (int64_t)device_cu_count() * 64;
  if (grid > maxgrid) grid = maxgrid;
  // rows of 3 x 8 / 16 / 32 chunks: three chunks per lane, two or more rows
  // side by side in a wave, no idle lane and no barrier
  if (const int l3 = lanes_per_row_x3(n2 / E)) {
    const int threads3 = 256;
    const int rpb3 = (threads3 / kWave) * (kWave / l3);
    int64_t grid3 = ceil_div(ceil_div(n1, rpb3), iters);
    if (grid3 > maxgrid) grid3 = maxgrid;
#define OSLO_FWD_X3(LPR_)                                                    \
  case LPR_:                                                                 \
    if constexpr (kCanFuse) {                                                \
      if (fused) {                                                           \
        norm_fwd_reg_kernel<T, V, 3, RMS, true, 256, true, LPR_>             \
            <<<dim3((unsigned)grid3), threads3, 0, st>>>(                    \
                (const T *)x, (const V *)gamma, (const V *)beta, (V *)y,     \
                mean, invvar, n1, (int)n2, eps, 1, rpb3, iters, *fp);        \
        break;                                                               \
      }                                                                      \
    }                                                                        \
    norm_fwd_reg_kernel<T, V, 3, RMS, true, 256, false, LPR_>                \
        <<<dim3((unsigned)grid3), threads3, 0, st>>>(                        \
            (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean,   \
            invvar, n1, (int)n2, eps, 1, rpb3, iters, FusePrologue{});       \
    break;
    switch (l3) {
      OSLO_FWD_X3(8)
      OSLO_FWD_X3(16)
      OSLO_FWD_X3(32)
    }
#undef OSLO_FWD_X3
    return check_launch("norm_fwd_reg_kernel (three chunks per lane)");
  }
  // short rows side by side in a wave
  const int lpr = (sp.wpr == 1 && sp.vpl == 1) ? lanes_per_row(n2 / E) : kWave;
  if (lpr < kWave) {
    // (these builds are bounded to 256 threads: at most four waves)
    const int waves_l = sp.rpb < 4 ? sp.rpb : 4;
    const int threads_l = kWave * waves_l;
    const int rpb_eff = waves_l * (kWave / lpr);
    const bool even_l = (n2 / E) == lpr;
    int64_t grid_l = ceil_div(ceil_div(n1, rpb_eff), iters);
    if (grid_l > maxgrid) grid_l = maxgrid;
    if constexpr (kCanFuse) {
      if (fused) {
#define OSLO_FWD_LPR_FUSED(LPR_)                                             \
  case LPR_:                                                                 \
    if (even_l)                                                              \
      norm_fwd_reg_kernel<T, V, 1, RMS, true, 256, true, LPR_>               \
          <<<dim3((unsigned)grid_l), threads_l, 0, st>>>(                      \
              (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean, \
              invvar, n1, (int)n2, eps, 1, rpb_eff, iters, *fp);             \
    else                                                                     \
      norm_fwd_reg_kernel<T, V, 1, RMS, false, 256, true, LPR_>              \
          <<<dim3((unsigned)grid_l), threads_l, 0, st>>>(                      \
              (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean, \
              invvar, n1, (int)n2, eps, 1, rpb_eff, iters, *fp);             \
    break;
        switch (lpr) {
          OSLO_FWD_LPR_FUSED(8)
          OSLO_FWD_LPR_FUSED(16)
          OSLO_FWD_LPR_FUSED(32)
        }
#undef OSLO_FWD_LPR_FUSED
        return check_launch("norm_fwd_reg_kernel (fused, side-by-side rows)");
      }
    }
#define OSLO_FWD_LPR(LPR_)                                                   \
  case LPR_:                                                                 \
    if (even_l)                                                              \
      norm_fwd_reg_kernel<T, V, 1, RMS, true, 256, false, LPR_>              \
          <<<dim3((unsigned)grid_l), threads_l, 0, st>>>(                      \
              (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean, \
              invvar, n1, (int)n2, eps, 1, rpb_eff, iters, FusePrologue{});  \
    else                                                                     \
      norm_fwd_reg_kernel<T, V, 1, RMS, false, 256, false, LPR_>             \
          <<<dim3((unsigned)grid_l), threads_l, 0, st>>>(                      \
              (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean, \
              invvar, n1, (int)n2, eps, 1, rpb_eff, iters, FusePrologue{});  \
    break;
    switch (lpr) {
      OSLO_FWD_LPR(8)
      OSLO_FWD_LPR(16)
      OSLO_FWD_LPR(32)
    }
#undef OSLO_FWD_LPR
    return check_launch("norm_fwd_reg_kernel (side-by-side rows)");
  }
  if constexpr (kCanFuse) {
    if (fused) {
#define OSLO_FWD_FUSED_L(VPL, EVEN_, MAXT_)                                 \
  norm_fwd_reg_kernel<T, V, VPL, RMS, EVEN_, MAXT_, true>                   \
      <<<dim3((unsigned)grid), threads, 0, st>>>(                           \
          (const T *)x, (const V *)gamma, (const V *)beta, (V *)y, mean,    \
          invvar, n1, (int)n2, eps, sp.wpr, sp.rpb, iters, *fp)
#define OSLO_FWD_FUSED(VPL)                                                 \
  case VPL:                                                                 \
    if constexpr (VPL * E <= 16) {                                          \
      if (!fused_big) {                                                     \
        if (even) OSLO_FWD_FUSED_L(VPL, true, 256);                         \
        else OSLO_FWD_FUSED_L(VPL, false, 256);                             \
      } else {                                                              \
        if (even) OSLO_FWD_FUSED_L(VPL, true, 1024);                        \
        else OSLO_FWD_FUSED_L(VPL, false, 1024);                            \
      }                                                                     \
      break;                                                                \
    }                                                                       \
    return fail(OSLO_ERR_UNSUPPORTED, "fused norm fwd: no kernel for vpl=%d", VPL);
      switch (sp.vpl) {
        OSLO_FWD_FUSED(1)
        OSLO_FWD_FUSED(2)
        OSLO_FWD_FUSED(4)
        default:
          return fail(OSLO_ERR_UNSUPPORTED, "fused norm fwd: no kernel for vpl=%d", sp.vpl);
      }
#undef OSLO_FWD_FUSED
#undef OSLO_FWD_FUSED_L
      return check_launch("norm_fwd_reg_kernel (fused)");
    }
  }
#define OSLO_FWD_CASE(VPL)                                                  \
  case VPL:                                                                 \
    if (threads <= 256 && even)                                             \
      norm_fwd_reg_kernel<T, V, VPL, RMS, true, 256>                        \
          <<<dim3((unsigned)grid), threads, 0, st>>>(                       \
              (const T *)x, (const V *)gamma, (const V *)beta, (V *)y,      \
              mean, invvar, n1, (int)n2, eps, sp.wpr, sp.rpb, iters, FusePrologue{});             \
    else if (threads <= 256)                                                \
      norm_fwd_reg_kernel<T, V, VPL, RMS, false, 256>                       \
          <<<dim3((unsigned)grid), threads, 0, st>>>(                       \
              (const T *)x, (const V *)gamma, (const V *)beta, (V *)y,      \
              mean, invvar, n1, (int)n2, eps, sp.wpr, sp.rpb, iters, FusePrologue{});             \
    else if constexpr (VPL * E <= 32) {                                     \
      if (even)                                                             \
        norm_fwd_reg_kernel<T, V, VPL, RMS, true, 1024>                     \
            <<<dim3((unsigned)grid), threads, 0, st>>>(                     \
                (const T *)x, (const V *)gamma, (const V *)beta, (V *)y,    \
                mean, invvar, n1, (int)n2, eps, sp.wpr, sp.rpb, iters, FusePrologue{});           \
      else                                                                  \
        norm_fwd_reg_kernel<T, V, VPL, RMS, false, 1024>                    \
            <<<dim3((unsigned)grid), threads, 0, st>>>(                     \
                (const T *)x, (const V *)gamma, (const V *)beta, (V *)y,    \
                mean, invvar, n1, (int)n2, eps, sp.wpr, sp.rpb, iters, FusePrologue{});           \
    }                                                                       \
    else                                                                    \
      return fail(OSLO_ERR_UNSUPPORTED,                                     \
                  "norm fwd: vpl=%d needs a workgroup of at most 256 "      \
                  "threads", VPL);                                          \
    break;
  switch (sp.vpl) {
    OSLO_FWD_CASE(1)
    OSLO_FWD_CASE(2)
    case 3:
      // (built for LayerNorm only, which is what selects it by default)
      if constexpr (!RMS) {
        switch (sp.vpl) { OSLO_FWD_CASE(3) }
        break;
      } else {
        return fail(OSLO_ERR_UNSUPPORTED, "norm fwd: three chunks per lane are built for LayerNorm only");
      }
    OSLO_FWD_CASE(4)
    OSLO_FWD_CASE(8)
    default:
      return fail(OSLO_ERR_UNSUPPORTED, "norm fwd: no kernel for vpl=%d", sp.vpl);
  }
#undef OSLO_FWD_CASE
  return check_launch("norm_fwd_reg_kernel");
}

// Column sums of a stored [rows, cols] tensor, one thread per column.
template <typename T>
__global__ __launch_bounds__(256) void norm_colsum_generic_kernel(
    const T *__restrict__ a, T *__restrict__ out, int64_t rows, int64_t cols) {
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= cols) return;
  float s = 0.f;
  for (int64_t r = 0; r < rows; ++r) s += io<T>::from_scalar(a[r * cols + col]);
  out[col] = io<T>::to_scalar(s);
}

// fe != nullptr selects the fused epilogue (T == V); dbias is then the bias
// gradient (may be null).
template <typename T, typename V, bool RMS>
static int launch_norm_bwd(const void *dy, const void *x, const float *mean,
                           const float *invvar, const void *gamma, void *dx,
                           void *dgamma, void *dbeta, void *ws,
                           int64_t ws_bytes, int64_t n1, int64_t n2,
                           hipStream_t st, const FuseEpilogue *fe = nullptr,
                           void *dbias = nullptr) {
  constexpr int E = chunk_elems<T, V>::value;
  constexpr int NARR = RMS ? 1 : 2;
  constexpr bool kCanFuse = sizeof(T) == sizeof(V);
  const bool fused = fe != nullptr;
  const bool want_params = dgamma != nullptr || (fused && dbias != nullptr);
  const bool vec_ok = n2 % E == 0 && aligned16(dy) && aligned16(x) &&
                      aligned16(dx) && aligned16(gamma) && aligned16(ws) &&
                      (!fused || (aligned16(fe->dh_extra) && aligned16(fe->dx_drop))) &&
                      n2 <= (int64_t)kWave * 16 * (16 / E) * E;
  // at most 16 elements per lane: 5 register arrays of that size stay
  // below the 128-VGPR budget of a 1024-thread workgroup
  static const int kVpl8[] = {1, 2};
  static const int kVpl4[] = {1, 2, 4};
  RowSplit sp{0, 1, 1, false};
  if (vec_ok) {
    const int *allowed = E == 8 ? kVpl8 : kVpl4;
    const int nallowed = E == 8 ? 2 : 3;
    const int waves = g_tune.norm_bwd_waves > 0 ? g_tune.norm_bwd_waves : 16;
    if (g_tune.norm_bwd_vpl > 0) {
      int cap = g_tune.norm_bwd_vpl;
      if (cap > 16 / E) cap = 16 / E;
      sp = split_row(n2 / E, cap, allowed, nallowed, waves);
    } else {
      // measured best on MI355X: 8 elements per lane wherever a row then
      // fits one workgroup, else 16 elements per lane
      sp = split_row(n2 / E, 8 / E, allowed, nallowed, waves);
      if (!sp.ok) {
        const RowSplit wide = split_row(n2 / E, 16 / E, allowed, nallowed, waves);
        if (wide.ok) sp = wide;
      }
    }
  }
  if (!sp.ok) {
    int64_t grid = n1 < 65535 * 16 ? n1 : 65535 * 16;
    norm_bwd_dx_generic_kernel<T, V, RMS><<<dim3((unsigned)grid), 256, 0, st>>>(
        (const V *)dy, (const T *)x, mean, invvar, (const V *)gamma, (T *)dx,
        n1, n2, fused ? *fe : FuseEpilogue{});
    int rc = check_launch("norm_bwd_dx_generic_kernel");
    if (rc != OSLO_OK) return rc;
    if constexpr (kCanFuse) {
      if (fused) {
        if (dbias != nullptr) {
          const void *src = fe->dx_drop != nullptr ? fe->dx_drop : dx;
          if (fe->drop && fe->dx_drop == nullptr)
            return fail(OSLO_ERR_INVALID_ARGUMENT,
                        "fused norm bwd: dbias with dropout needs dx_drop");
          const int64_t S = generic_colsum_slices(ws, ws_bytes, 1, n1, n2);
          if (S > 0) {
            StoredValue<T> f{(const T *)src, n2};
            rc = launch_generic_colsum<1, T>(f, ws, S, n1, n2, dbias, nullptr, st);
          } else {
            norm_colsum_generic_kernel<T>
                <<<dim3((unsigned)ceil_div(n2, 256)), 256, 0, st>>>(
                    (const T *)src, (T *)dbias, n1, n2);
            rc = check_launch("norm_colsum_generic_kernel");
          }
          if (rc != OSLO_OK) return rc;
        }
      }
    }
    if (dgamma == nullptr) return rc;
    {
      // (stream order: the partial rows of a bias gradient above have been
      //  consumed by their own finalize before these overwrite them)
      constexpr int NA = RMS ? 1 : 2;
      const int64_t S = generic_colsum_slices(ws, ws_bytes, NA, n1, n2);
      if (S > 0) {
        NormParamGrad<T, V, RMS> f{(const V *)dy, (const T *)x, mean, invvar, n2};
        return launch_generic_colsum<NA, V>(f, ws, S, n1, n2, dgamma, dbeta, st);
      }
    }
    norm_bwd_param_generic_kernel<T, V, RMS>
        <<<dim3((unsigned)ceil_div(n2, 256)), 256, 0, st>>>(
            (const V *)dy, (const T *)x, mean, invvar, (V *)dgamma,
            (V *)dbeta, n1, n2);
    return check_launch("norm_bwd_param_generic_kernel");
  }
  // rows that are a whole number of half-waves but not of waves (96, 160 or
  // 224 chunks: 768, 1280, 1792 16-bit elements): units of 32 lanes, so that
  // no lane idles
  int upr = 0;
  if (E == 8 && g_tune.norm_lanes_per_row != kWave && sp.vpl == 1) {
    const int64_t nch = n2 / E;
    if (nch % 32 == 0 && nch % 64 != 0 && (nch == 96 || nch == 160 || nch == 224))
      upr = (int)(nch / 32);
  }
  if (upr > 0) {
    sp.wpr = upr;
    sp.rpb = 32 / upr;
  }
  // short rows side by side in a wave: the row slots of a workgroup multiply
  // (the three-chunks-per-lane mapping of the forward kernel does not pay
  //  here: its 24 elements per lane and operand need a 512-thread workgroup,
  //  and eight waves per CU measure 2 % slower than whole-wave rows)
  const int lpr = (sp.wpr == 1 && sp.vpl == 1) ? lanes_per_row(n2 / E) : kWave;
  const int wave_slots = sp.rpb;  // row slots at wave granularity
  if (lpr < kWave) sp.rpb *= kWave / lpr;
  int64_t P = colsum_parts_norm(n1, n2);
  if (P > ceil_div(n1, sp.rpb)) P = ceil_div(n1, sp.rpb);
  float *part = nullptr;
  FuseEpilogue fev{};
  if (fused) {
    fev = *fe;
    fev.want_dbias = dbias != nullptr ? 1 : 0;
  }
  const int narr = NARR + (fev.want_dbias ? 1 : 0);
  if (want_params) {
    const int64_t need = (int64_t)narr * P * n2 * (int64_t)sizeof(float);
    if (ws == nullptr || ws_bytes < need)
      return fail(OSLO_ERR_WORKSPACE,
                  "norm bwd: workspace of %lld bytes needed, %lld given",
                  (long long)need, (long long)ws_bytes);
    part = (float *)ws;
  }
  const int threads = (upr > 0 ? 32 : kWave) * sp.wpr * wave_slots;
  // LDS: one row of column partials when a workgroup holds several row
  // slots, and behind it the chunks of gamma that 16 elements per lane move
  // out of the registers (one of four with 4-byte parameters, else all)
  size_t lds = wave_slots > 1 ? (size_t)n2 * sizeof(float) : 0;
  if (sp.vpl * E >= 16)
    lds += (size_t)(sp.vpl - (sizeof(V) == 4 ? 1 : 0)) * threads * E * sizeof(V);
  const bool even = upr > 0 ? true
                  : lpr < kWave ? (n2 / E) == lpr
                                : (n2 / E) == (int64_t)sp.vpl * kWave * sp.wpr;
  // rows in flight ahead of the one being reduced: two while the packed row
  // buffers are small (8 elements per lane) and a row spans several waves,
  // else one (a wave that owns whole rows measures 6 % slower with two)
  // (plain workgroups of twelve waves, rows of 3072 and 6144 16-bit
  //  elements, measure 2.5 % faster with one; with the fused epilogue 8 %
  //  slower)
  int pf = sp.vpl * E <= 8 && sp.wpr >= 2 && (fused || threads != 12 * kWave) ? 2 : 1;
  if (g_tune.norm_bwd_prefetch > 0) pf = g_tune.norm_bwd_prefetch >= 2 ? 2 : 1;
#define OSLO_BWD_LAUNCH_T(VPL, EVEN_, PF_, MAXT_)                          \
  do {                                                                     \
    if constexpr (kCanFuse) {                                              \
      if (fused) {                                                         \
        norm_bwd_reg_kernel<T, V, VPL, RMS, EVEN_, PF_, true, MAXT_>       \
            <<<dim3((unsigned)P), threads, lds, st>>>(                     \
                (const V *)dy, (const T *)x, mean, invvar,                 \
                (const V *)gamma, (T *)dx, part, n1, (int)n2, sp.wpr,      \
                sp.rpb, fev);                                              \
        break;                                                             \
      }                                                                    \
    }                                                                      \
    norm_bwd_reg_kernel<T, V, VPL, RMS, EVEN_, PF_, false, MAXT_>          \
        <<<dim3((unsigned)P), threads, lds, st>>>(                         \
            (const V *)dy, (const T *)x, mean, invvar, (const V *)gamma,   \
            (T *)dx, part, n1, (int)n2, sp.wpr, sp.rpb, fev);              \
  } while (0)
  // the 16-elements-per-lane builds exist for 768 threads as well
#define OSLO_BWD_LAUNCH(VPL, EVEN_, PF_)                                   \
  do {                                                                     \
    if constexpr (VPL * E == 16) {                                         \
      if (threads <= 768) {                                                \
        OSLO_BWD_LAUNCH_T(VPL, EVEN_, PF_, 768);                           \
        break;                                                             \
      }                                                                    \
    }                                                                      \
    OSLO_BWD_LAUNCH_T(VPL, EVEN_, PF_, 1024);                              \
  } while (0)
#define OSLO_BWD_CASE(VPL)                                                 \
  case VPL:                                                                \
    if constexpr (VPL * E <= 16) {                                         \
      if (even && pf == 2)                                                 \
        OSLO_BWD_LAUNCH(VPL, true, 2);                                     \
      else if (even)                                                       \
        OSLO_BWD_LAUNCH(VPL, true, 1);                                     \
      else if (pf == 2)                                                    \
        OSLO_BWD_LAUNCH(VPL, false, 2);                                    \
      else                                                                 \
        OSLO_BWD_LAUNCH(VPL, false, 1);                                    \
    }                                                                      \
    break;
  if (upr > 0) {
#define OSLO_BWD_UNIT(PF_)                                                  \
  do {                                                                      \
    if constexpr (kCanFuse) {                                               \
      if (fused) {                                                          \
        norm_bwd_reg_kernel<T, V, 1, RMS, true, PF_, true, 1024, kWave, 32> \
            <<<dim3((unsigned)P), threads, lds, st>>>(                      \
                (const V *)dy, (const T *)x, mean, invvar,                  \
                (const V *)gamma, (T *)dx, part, n1, (int)n2, sp.wpr,       \
                sp.rpb, fev);                                               \
        break;                                                              \
      }                                                                     \
    }                                                                       \
    norm_bwd_reg_kernel<T, V, 1, RMS, true, PF_, false, 1024, kWave, 32>    \
        <<<dim3((unsigned)P), threads, lds, st>>>(                          \
            (const V *)dy, (const T *)x, mean, invvar, (const V *)gamma,    \
            (T *)dx, part, n1, (int)n2, sp.wpr, sp.rpb, fev);               \
  } while (0)
    if constexpr (E == 8) {
      if (pf == 2) OSLO_BWD_UNIT(2);
      else OSLO_BWD_UNIT(1);
    }
#undef OSLO_BWD_UNIT
  } else if (lpr < kWave) {
#define OSLO_BWD_LPR(LPR_)                                                  \
  case LPR_:                                                                \
    if constexpr (kCanFuse) {                                               \
      if (fused) {                                                          \
        if (even)                                                           \
          norm_bwd_reg_kernel<T, V, 1, RMS, true, 1, true, 1024, LPR_>      \
              <<<dim3((unsigned)P), threads, lds, st>>>(                    \
                  (const V *)dy, (const T *)x, mean, invvar,                \
                  (const V *)gamma, (T *)dx, part, n1, (int)n2, 1, sp.rpb,  \
                  fev);                                                     \
        else                                                                \
          norm_bwd_reg_kernel<T, V, 1, RMS, false, 1, true, 1024, LPR_>     \
              <<<dim3((unsigned)P), threads, lds, st>>>(                    \
                  (const V *)dy, (const T *)x, mean, invvar,                \
                  (const V *)gamma, (T *)dx, part, n1, (int)n2, 1, sp.rpb,  \
                  fev);                                                     \
        break;                                                              \
      }                                                                     \
    }                                                                       \
    if (even)                                                               \
      norm_bwd_reg_kernel<T, V, 1, RMS, true, 1, false, 1024, LPR_>         \
          <<<dim3((unsigned)P), threads, lds, st>>>(                        \
              (const V *)dy, (const T *)x, mean, invvar, (const V *)gamma,  \
              (T *)dx, part, n1, (int)n2, 1, sp.rpb, fev);                  \
    else                                                                    \
      norm_bwd_reg_kernel<T, V, 1, RMS, false, 1, false, 1024, LPR_>        \
          <<<dim3((unsigned)P), threads, lds, st>>>(                        \
              (const V *)dy, (const T *)x, mean, invvar, (const V *)gamma,  \
              (T *)dx, part, n1, (int)n2, 1, sp.rpb, fev);                  \
    break;
    switch (lpr) {
      OSLO_BWD_LPR(8)
      OSLO_BWD_LPR(16)
      OSLO_BWD_LPR(32)
    }
#undef OSLO_BWD_LPR
  } else
  switch (sp.vpl) {
    OSLO_BWD_CASE(1)
    OSLO_BWD_CASE(2)
    OSLO_BWD_CASE(4)
    default:
      return fail(OSLO_ERR_UNSUPPORTED, "norm bwd: no kernel for vpl=%d", sp.vpl);
  }
#undef OSLO_BWD_LAUNCH
#undef OSLO_BWD_LAUNCH_T
#undef OSLO_BWD_CASE
  int rc = check_launch("norm_bwd_reg_kernel");
  if (rc != OSLO_OK || !want_params) return rc;
  if (g_tune.colsum_defer) return rc;  // measurement only: see oslo_colsum_finalize_probe
  // arrays of partial rows: dgamma, dbeta (LayerNorm), bias gradient (fused)
  void *outs[3] = {dgamma, nullptr, nullptr};
  int na = 1;
  if (!RMS) outs[na++] = dbeta;
  if (fev.want_dbias) outs[na++] = dbias;
  return launch_colsum_finalize<V>(part, P, n2, outs[0], outs[1], st, outs[2], na);
}

// Zero fill of a small parameter-gradient vector (a kernel rather than a
// memset node, so that a caller may capture the call in a HIP graph).
__global__ __launch_bounds__(256) void zero_bytes_kernel(uint8_t *p, int64_t nbytes) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nbytes;
       i += (int64_t)gridDim.x * 256)
    p[i] = 0;
}

static int zero_params(void *p, int64_t nbytes, hipStream_t st) {
  if (p == nullptr || nbytes <= 0) return OSLO_OK;
  int64_t grid = ceil_div(nbytes, 256);
  if (grid > 1024) grid = 1024;
  zero_bytes_kernel<<<dim3((unsigned)grid), 256, 0, st>>>((uint8_t *)p, nbytes);
  return check_launch("zero_bytes_kernel");
}

static int check_norm_dtypes(int din, int dout) {
  if (din == OSLO_DTYPE_F64 || dout == OSLO_DTYPE_F64) {
    if (din == dout) return OSLO_OK;
    return fail(OSLO_ERR_UNSUPPORTED,
                "dtype pair (in=%d, out=%d) unsupported: double input and "
                "double output go together",
                din, dout);
  }
  if (!valid_dtype(din) || !valid_dtype(dout))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "unknown dtype (%d, %d)", din, dout);
  if (din != OSLO_DTYPE_F32 && din != dout)
    return fail(OSLO_ERR_UNSUPPORTED,
                "dtype pair (in=%d, out=%d) unsupported: a 16-bit input "
                "requires the same output type",
                din, dout);
  return OSLO_OK;
}

// Expands to a call of FN<T, V, RMS> for the allowed dtype pairs.
#define OSLO_NORM_DISPATCH(din, dout, RMS, FN, ...)                          \
  do {                                                                       \
    if (din == OSLO_DTYPE_F32 && dout == OSLO_DTYPE_F32)                     \
      return FN<float, float, RMS>(__VA_ARGS__);                             \
    if (din == OSLO_DTYPE_F32 && dout == OSLO_DTYPE_F16)                     \
      return FN<float, _Float16, RMS>(__VA_ARGS__);                          \
    if (din == OSLO_DTYPE_F32 && dout == OSLO_DTYPE_BF16)                    \
      return FN<float, __bf16, RMS>(__VA_ARGS__);                            \
    if (din == OSLO_DTYPE_F16) return FN<_Float16, _Float16, RMS>(__VA_ARGS__); \
    return FN<__bf16, __bf16, RMS>(__VA_ARGS__);                             \
  } while (0)

static int norm_fwd_entry(bool rms, const void *x, const void *gamma,
                          const void *beta, void *y, void *mean_,
                          void *invvar_, int64_t n1, int64_t n2, double eps,
                          int din, int dout, void *stream) {
  int rc = check_norm_dtypes(din, dout);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(n1 >= 0 && n2 >= 1, "norm fwd: bad shape [%lld, %lld]",
               (long long)n1, (long long)n2);
  OSLO_REQUIRE(n2 <= 0x7fffffff, "norm fwd: n2 too large");
  if (n1 == 0) return OSLO_OK;
  OSLO_REQUIRE(x && y && invvar_, "norm fwd: null tensor pointer");
  OSLO_REQUIRE(rms || mean_, "layer norm fwd: null mean pointer");
  OSLO_REQUIRE(rms || (gamma == nullptr) == (beta == nullptr),
               "layer norm fwd: gamma and beta must both be given or both be "
               "NULL");
  hipStream_t st = (hipStream_t)stream;
  if (din == OSLO_DTYPE_F64)
    return launch_norm_f64_fwd(rms, x, gamma, beta, y, mean_, invvar_, n1, n2,
                               eps, st);
  float *mean = static_cast<float *>(mean_);
  float *invvar = static_cast<float *>(invvar_);
  if (rms)
    OSLO_NORM_DISPATCH(din, dout, true, launch_norm_fwd, x, gamma, nullptr, y,
                       nullptr, invvar, n1, n2, (float)eps, st);
  OSLO_NORM_DISPATCH(din, dout, false, launch_norm_fwd, x, gamma, beta, y,
                     mean, invvar, n1, n2, (float)eps, st);
}

static int norm_bwd_entry(bool rms, const void *dy, const void *x,
                          const void *mean_, const void *invvar_,
                          const void *gamma, void *dx, void *dgamma,
                          void *dbeta, void *ws, int64_t ws_bytes, int64_t n1,
                          int64_t n2, int din, int dout, void *stream) {
  int rc = check_norm_dtypes(din, dout);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(n1 >= 0 && n2 >= 1, "norm bwd: bad shape [%lld, %lld]",
               (long long)n1, (long long)n2);
  OSLO_REQUIRE(n2 <= 0x7fffffff, "norm bwd: n2 too large");
  OSLO_REQUIRE(gamma != nullptr || dgamma == nullptr,
               "norm bwd: dgamma requested without gamma");
  OSLO_REQUIRE(rms || (dgamma == nullptr) == (dbeta == nullptr),
               "layer norm bwd: dgamma and dbeta must both be given or both be "
               "NULL");
  if (n1 == 0) {
    // an empty batch still defines zero parameter gradients
    hipStream_t st0 = (hipStream_t)stream;
    int rc0 = zero_params(dgamma, n2 * dtype_size(dout), st0);
    if (rc0 == OSLO_OK) rc0 = zero_params(dbeta, n2 * dtype_size(dout), st0);
    return rc0;
  }
  OSLO_REQUIRE(dy && x && invvar_ && dx, "norm bwd: null tensor pointer");
  OSLO_REQUIRE(rms || mean_, "layer norm bwd: null mean pointer");
  hipStream_t st = (hipStream_t)stream;
  if (din == OSLO_DTYPE_F64)
    return launch_norm_f64_bwd(rms, dy, x, mean_, invvar_, gamma, dx, dgamma,
                               dbeta, n1, n2, st);
  const float *mean = static_cast<const float *>(mean_);
  const float *invvar = static_cast<const float *>(invvar_);
  if (rms)
    OSLO_NORM_DISPATCH(din, dout, true, launch_norm_bwd, dy, x, nullptr, invvar,
                       gamma, dx, dgamma, nullptr, ws, ws_bytes, n1, n2, st);
  OSLO_NORM_DISPATCH(din, dout, false, launch_norm_bwd, dy, x, mean, invvar,
                     gamma, dx, dgamma, dbeta, ws, ws_bytes, n1, n2, st);
}

// ---------------------------------------------------------------------------
// LayerNorm backward without a workspace argument: the fp32 partial rows of
// dgamma / dbeta live in a file-scope device array.  Every GPU holds its own
// copy of the array at its own address; in host code the array's name is only
// a handle for hipGetSymbolAddress, never a device address.
// ---------------------------------------------------------------------------
constexpr int64_t kStaticScratchBytes = OSLO_LN_BWD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per
// device (threads that race here obtain the same address).
static int static_scratch(void **out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail(OSLO_ERR_LAUNCH, "ln bwd static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(OSLO_ERR_UNSUPPORTED, "ln bwd static: device index %d beyond %d", dev,
                kMaxDevices - 1);
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(OSLO_ERR_LAUNCH, "ln bwd static: hipGetSymbolAddress: %s",
                  hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return OSLO_OK;
}

}  // namespace oslo

extern "C" {

int oslo_ln_fwd(const void *x, const void *gamma, const void *beta, void *y,
                void *mean, void *invvar, int64_t n1, int64_t n2, double eps,
                int dtype_in, int dtype_out, void *stream) {
  oslo::tune_snapshot();
  return oslo::norm_fwd_entry(false, x, gamma, beta, y, mean, invvar, n1, n2,
                              eps, dtype_in, dtype_out, stream);
}

int oslo_rms_fwd(const void *x, const void *gamma, void *y, void *invvar,
                 int64_t n1, int64_t n2, double eps, int dtype_in,
                 int dtype_out, void *stream) {
  oslo::tune_snapshot();
  return oslo::norm_fwd_entry(true, x, gamma, nullptr, y, nullptr, invvar, n1,
                              n2, eps, dtype_in, dtype_out, stream);
}

int oslo_ln_bwd(const void *dy, const void *x, const void *mean,
                const void *invvar, const void *gamma, void *dx, void *dgamma,
                void *dbeta, void *workspace, int64_t workspace_bytes,
                int64_t n1, int64_t n2, int dtype_in, int dtype_out,
                void *stream) {
  oslo::tune_snapshot();
  return oslo::norm_bwd_entry(false, dy, x, mean, invvar, gamma, dx, dgamma,
                              dbeta, workspace, workspace_bytes, n1, n2,
                              dtype_in, dtype_out, stream);
}

int oslo_rms_bwd(const void *dy, const void *x, const void *invvar,
                 const void *gamma, void *dx, void *dgamma, void *workspace,
                 int64_t workspace_bytes, int64_t n1, int64_t n2, int dtype_in,
                 int dtype_out, void *stream) {
  oslo::tune_snapshot();
  return oslo::norm_bwd_entry(true, dy, x, nullptr, invvar, gamma, dx, dgamma,
                              nullptr, workspace, workspace_bytes, n1, n2,
                              dtype_in, dtype_out, stream);
}

int oslo_ln_bwd_static(const void *dy, const void *x, const void *mean,
                       const void *invvar, const void *gamma, void *dx,
                       void *dgamma, void *dbeta, int64_t n1, int64_t n2,
                       int dtype_in, int dtype_out, void *stream) {
  oslo::tune_snapshot();
  using namespace oslo;
  OSLO_REQUIRE(n1 >= 0 && n2 >= 1, "ln bwd static: bad shape [%lld, %lld]",
               (long long)n1, (long long)n2);
  void *ws = nullptr;
  if (dgamma != nullptr && n1 > 0 && dtype_in != OSLO_DTYPE_F64) {
    const int64_t need = oslo_workspace_bytes(OSLO_OP_LN_BWD, n1, n2);
    if (need < 0) return (int)need;
    if (need > kStaticScratchBytes)
      return fail(OSLO_ERR_WORKSPACE,
                  "ln bwd static: [%lld, %lld] needs %lld bytes of partial rows, "
                  "the static scratch holds %lld; use oslo_ln_bwd with a "
                  "workspace",
                  (long long)n1, (long long)n2, (long long)need,
                  (long long)kStaticScratchBytes);
    const int rc = static_scratch(&ws);
    if (rc != OSLO_OK) return rc;
  }
  // The partial rows are written in full before the finalize kernel reads
  // them: nothing in the array has to start at zero.
  return norm_bwd_entry(false, dy, x, mean, invvar, gamma, dx, dgamma, dbeta, ws,
                        ws != nullptr ? kStaticScratchBytes : 0, n1, n2,
                        dtype_in, dtype_out, stream);
}

int oslo_bias_dropout_add_norm_fwd(const void *x, const void *bias,
                                   const void *residual, const void *gamma,
                                   const void *beta, void *h_out, void *y,
                                   float *mean, float *invvar, int64_t n1,
                                   int64_t n2, double eps, float p,
                                   uint64_t seed, uint64_t offset, int rms,
                                   int dtype, void *stream) {
  oslo::tune_snapshot();
  using namespace oslo;
  int rc = check_norm_dtypes(dtype, dtype);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(n1 >= 0 && n2 >= 1 && n2 <= 0x7fffffff,
               "fused norm fwd: bad shape [%lld, %lld]", (long long)n1,
               (long long)n2);
  OSLO_REQUIRE(p >= 0.f && p <= 1.f, "fused norm fwd: p = %g outside [0, 1]",
               (double)p);
  if (n1 == 0) return OSLO_OK;
  OSLO_REQUIRE(x && y && invvar, "fused norm fwd: null tensor pointer");
  OSLO_REQUIRE(rms || mean, "fused layer norm fwd: null mean pointer");
  OSLO_REQUIRE(rms || (gamma == nullptr) == (beta == nullptr),
               "fused layer norm fwd: gamma and beta must both be given or "
               "both be NULL");
  hipStream_t st = (hipStream_t)stream;
  FusePrologue fp{bias, residual, h_out, make_drop(p, seed, offset),
                  p > 0.f ? 1 : 0};
  if (rms) beta = nullptr;
#define OSLO_FUSED_FWD(T_)                                                    \
  (rms ? launch_norm_fwd<T_, T_, true>(x, gamma, nullptr, y, nullptr, invvar, \
                                       n1, n2, (float)eps, st, &fp)           \
       : launch_norm_fwd<T_, T_, false>(x, gamma, beta, y, mean, invvar, n1,  \
                                        n2, (float)eps, st, &fp))
  rc = dtype == OSLO_DTYPE_F32   ? OSLO_FUSED_FWD(float)
       : dtype == OSLO_DTYPE_F16 ? OSLO_FUSED_FWD(_Float16)
                                 : OSLO_FUSED_FWD(__bf16);
#undef OSLO_FUSED_FWD
  if (rc != kNotFused) return rc;
  // Rows outside the register path: the same arithmetic as two launches, h
  // staged in h_out (or in y, which the norm then overwrites in place).
  void *buf = h_out != nullptr ? h_out : y;
  rc = oslo_bias_dropout_add_fwd(x, bias, residual, buf, nullptr, n1, n2, p,
                                 seed, offset, dtype, stream);
  if (rc != OSLO_OK) return rc;
  return norm_fwd_entry(rms != 0, buf, gamma, beta, y, mean, invvar, n1, n2,
                        eps, dtype, dtype, stream);
}

int oslo_bias_dropout_add_norm_bwd(const void *dy, const void *dh_extra,
                                   const void *h, const float *mean,
                                   const float *invvar, const void *gamma,
                                   void *dres, void *dx, void *dgamma,
                                   void *dbeta, void *dbias, void *workspace,
                                   int64_t workspace_bytes, int64_t n1,
                                   int64_t n2, float p, uint64_t seed,
                                   uint64_t offset, int rms, int dtype,
                                   void *stream) {
  oslo::tune_snapshot();
  using namespace oslo;
  int rc = check_norm_dtypes(dtype, dtype);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(n1 >= 0 && n2 >= 1 && n2 <= 0x7fffffff,
               "fused norm bwd: bad shape [%lld, %lld]", (long long)n1,
               (long long)n2);
  OSLO_REQUIRE(p >= 0.f && p <= 1.f, "fused norm bwd: p = %g outside [0, 1]",
               (double)p);
  OSLO_REQUIRE(gamma != nullptr || dgamma == nullptr,
               "fused norm bwd: dgamma requested without gamma");
  OSLO_REQUIRE(rms || (dgamma == nullptr) == (dbeta == nullptr),
               "fused layer norm bwd: dgamma and dbeta must both be given or "
               "both be NULL");
  OSLO_REQUIRE(p == 0.f || dx != nullptr,
               "fused norm bwd: with dropout the gradient of x needs its own "
               "tensor (dx)");
  hipStream_t st = (hipStream_t)stream;
  if (n1 == 0) {
    const int64_t nb = n2 * dtype_size(dtype);
    rc = zero_params(dgamma, nb, st);
    if (rc == OSLO_OK && !rms) rc = zero_params(dbeta, nb, st);
    if (rc == OSLO_OK) rc = zero_params(dbias, nb, st);
    return rc;
  }
  OSLO_REQUIRE(dy && h && invvar && dres, "fused norm bwd: null tensor pointer");
  OSLO_REQUIRE(rms || mean, "fused layer norm bwd: null mean pointer");
  FuseEpilogue fe{dh_extra, dx, make_drop(p, seed, offset), p > 0.f ? 1 : 0, 0};
#define OSLO_FUSED_BWD(T_)                                                     \
  (rms ? launch_norm_bwd<T_, T_, true>(dy, h, nullptr, invvar, gamma, dres,    \
                                       dgamma, nullptr, workspace,             \
                                       workspace_bytes, n1, n2, st, &fe,       \
                                       dbias)                                  \
       : launch_norm_bwd<T_, T_, false>(dy, h, mean, invvar, gamma, dres,      \
                                        dgamma, dbeta, workspace,              \
                                        workspace_bytes, n1, n2, st, &fe,      \
                                        dbias))
  return dtype == OSLO_DTYPE_F32   ? OSLO_FUSED_BWD(float)
         : dtype == OSLO_DTYPE_F16 ? OSLO_FUSED_BWD(_Float16)
                                   : OSLO_FUSED_BWD(__bf16);
#undef OSLO_FUSED_BWD
}

}  // extern "C"
