// bias-GeLU (tanh approximation) and bias-dropout-add, forward and backward,
// plus the Philox test hooks, for gfx950.
//
// Thread mapping (all vector kernels): a lane owns one chunk of 8 consecutive
// columns.  A 256-thread workgroup is tx lanes wide (64, 128 or 256: up to
// 2048 columns, one contiguous 4 KB piece of a row) and ty = 256 / tx rows
// tall.  The rows are cut into steps of ty * U consecutive rows (a lane keeps
// U independent 128-bit loads in flight); workgroups are numbered column tile
// first, then slot, and slot s visits steps s, s + slots, s + 2 slots, ...
// Forward kernels launch one workgroup per step, so the launch sweeps memory
// front to back with short-lived waves.  Backward kernels launch about three
// workgroups per CU; they advance through the rows in lockstep (one compact
// moving window), keep the column sums of dx for their 8 columns in registers,
// fold the ty rows through LDS and write one fp32 partial row per slot, which
// colsum_finalize_kernel reduces deterministically.
//
// Formulas: oslo/torch/nn/modules/functional.py:23-50 (GeLU forward and
// derivative with the constants 0.79788456, 0.044715, 0.1070322243),
// :295-298 (dropout(x + bias)).
#include "capi.h"
#include "colsum.hip.h"
#include "common.hip.h"

namespace oslo {

// A chunk is one 128-bit vector: 8 elements of a 16-bit type, 4 of fp32 (kE
// inside the kernels).  The dropout groups are 8 consecutive elements of the
// flattened tensor for every dtype: an fp32 chunk takes half a group.

// -2 * log2(e) * 0.79788456 and that times 0.044715: exp(-2 z) = exp2(u * (K1 + K2 u^2))
constexpr float kGeluK1 = -2.0f * 1.4426950408889634f * 0.79788456f;
constexpr float kGeluK2 = kGeluK1 * 0.044715f;

// gelu(u) = u * sigmoid(2 z), z = 0.79788456 u (1 + 0.044715 u^2); identical
// to u * 0.5 * (1 + tanh z) without the cancellation of 1 + tanh for u << 0.
__device__ __forceinline__ float gelu_fwd(float u) {
  const float e = __builtin_amdgcn_exp2f(u * (kGeluK1 + kGeluK2 * u * u));
  return u * __builtin_amdgcn_rcpf(1.0f + e);
}

// d gelu / du = 0.5 u (1 - t^2)(0.79788456 + 0.1070322243 u^2) + 0.5 (1 + t)
// with t = tanh z; in terms of s = sigmoid(2 z), e = exp(-2 z):
// 1 + t = 2 s and 1 - t^2 = 4 e s^2.
// Evaluated as s + (u s (1 - s)) q with q = 2 * 0.79788456 + 2 * 0.1070322243 u^2
// and e s^2 = s (1 - s) formed by one fused multiply-add: eight instructions
// and two transcendentals.  e itself is never multiplied, so it may overflow:
// for u << 0 it becomes inf, s and the product term exact zeros, as tanh = -1
// makes them in the reference's form; the result is finite as long as u^2 is.
// (Where s rounds to 1 the product term, of relative size below 1e-6, is
// dropped; elsewhere the form is good to a few 1e-6.)
__device__ __forceinline__ float gelu_bwd(float u) {
  const float u2 = u * u;
  const float e = __builtin_amdgcn_exp2f(u * __builtin_fmaf(kGeluK2, u2, kGeluK1));
  const float s = __builtin_amdgcn_rcpf(1.0f + e);
  const float t = __builtin_fmaf(-s, s, s);
  const float q = __builtin_fmaf(2.0f * 0.1070322243f, u2, 2.0f * 0.79788456f);
  return __builtin_fmaf(u * t, q, s);
}

struct EltGeom {
  int64_t rows;
  int64_t cols;
  int nchunks;  // cols / 8
  int tx;       // lanes along the columns per workgroup: 64, 128 or 256
  int ty;       // 256 / tx rows side by side
  int tiles;    // column tiles = ceil(nchunks / tx)
  int64_t slots;  // workgroups per column tile; slot s visits row steps
                  // s, s + slots, s + 2 slots, ... of ty * U rows each
  // index of the launch's first workgroup among those of the whole problem (a
  // forward problem beyond 2^32 work-items takes several launches)
  int64_t blk0 = 0;
};

// Position of this thread: column chunk cc (may be >= nchunks), its row
// inside a step and the slot of its workgroup.  All workgroups advance through
// the rows together, so at any time the launch touches one compact window of
// memory that moves front to back.
struct EltPos {
  int cc, ry;
  int64_t slot;
};
__device__ __forceinline__ EltPos elt_pos(const EltGeom &g) {
  const int64_t b = (int64_t)blockIdx.x + g.blk0;
  EltPos p;
  p.slot = b / g.tiles;
  p.cc = (int)(b - p.slot * g.tiles) * g.tx + (int)(threadIdx.x % g.tx);
  p.ry = threadIdx.x / g.tx;
  return p;
}

template <typename T, int U, bool HAS_BIAS>
__global__ __launch_bounds__(256) void bias_gelu_fwd_kernel(
    const T *__restrict__ x, const T *__restrict__ bias, T *__restrict__ y,
    EltGeom g) {
  constexpr int kE = io<T>::EPV;
  const EltPos ps = elt_pos(g);
  if (ps.cc >= g.nchunks) return;
  float b[kE];
  if constexpr (HAS_BIAS) load_chunk<T, kE, false>(bias + (int64_t)ps.cc * kE, b);
  const int64_t coff = (int64_t)ps.cc * kE;
  for (int64_t r0 = ps.slot * g.ty * U + ps.ry; r0 < g.rows;
       r0 += g.slots * g.ty * U) {
    float v[U][kE];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = r0 + u * g.ty;
      if (r < g.rows) load_chunk<T, kE>(x + r * g.cols + coff, v[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = r0 + u * g.ty;
      if (r < g.rows) {
        float o[kE];
#pragma unroll
        for (int e = 0; e < kE; ++e)
          o[e] = gelu_fwd(HAS_BIAS ? v[u][e] + b[e] : v[u][e]);
        store_chunk<T, kE>(y + r * g.cols + coff, o);
      }
    }
  }
}

// Folds the per-lane column sums of the ty rows of the workgroup and writes
// the partial row of this slot.  sh is [ty][kE][tx] floats (at most 8 KB).
template <int kE>
__device__ __forceinline__ void write_col_partials(const float *acc, float *sh,
                                                   float *__restrict__ part,
                                                   const EltGeom &g,
                                                   const EltPos &ps) {
  const int cx = threadIdx.x % g.tx;
  const int ry = threadIdx.x / g.tx;
#pragma unroll
  for (int e = 0; e < kE; ++e) sh[(ry * kE + e) * g.tx + cx] = acc[e];
  __syncthreads();
  if (ry == 0 && ps.cc < g.nchunks) {
    float o[kE];
#pragma unroll
    for (int e = 0; e < kE; ++e) {
      float s = sh[e * g.tx + cx];
      for (int q = 1; q < g.ty; ++q) s += sh[(q * kE + e) * g.tx + cx];
      o[e] = s;
    }
    store_chunk<float, kE>(part + ps.slot * g.cols + (int64_t)ps.cc * kE, o);
  }
}

template <typename T, int U, bool HAS_BIAS>
__global__ __launch_bounds__(256) void bias_gelu_bwd_kernel(
    const T *__restrict__ gr, const T *__restrict__ x,
    const T *__restrict__ bias, T *__restrict__ dx, float *__restrict__ part,
    EltGeom g) {
  constexpr int kE = io<T>::EPV;
  __shared__ float sh[256 * kE];
  const EltPos ps = elt_pos(g);
  float b[kE], acc[kE];
#pragma unroll
  for (int e = 0; e < kE; ++e) {
    b[e] = 0.f;
    acc[e] = 0.f;
  }
  if (ps.cc < g.nchunks) {
    if constexpr (HAS_BIAS) load_chunk<T, kE, false>(bias + (int64_t)ps.cc * kE, b);
    const int64_t coff = (int64_t)ps.cc * kE;
    // The loads of the next step are requested, in packed form, before the
    // current step is evaluated; a row past the end re-reads the last row.
    RawChunk<T, kE> nx[U], ng[U];
    auto fetch = [&](int64_t r0) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int64_t r = r0 + u * g.ty;
        r = r < g.rows ? r : g.rows - 1;
        nx[u].load(x + r * g.cols + coff);
        ng[u].load(gr + r * g.cols + coff);
      }
    };
    const int64_t step = g.slots * g.ty * U;
    int64_t r0 = ps.slot * g.ty * U + ps.ry;
    if (r0 < g.rows) fetch(r0);
    for (; r0 < g.rows; r0 += step) {
      float v[U][kE], gv[U][kE];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        nx[u].unpack(v[u]);
        ng[u].unpack(gv[u]);
      }
      if (r0 + step < g.rows) fetch(r0 + step);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t r = r0 + u * g.ty;
        if (r < g.rows) {
          float o[kE];
#pragma unroll
          for (int e = 0; e < kE; ++e) o[e] = gelu_bwd(v[u][e] + b[e]) * gv[u][e];
          store_chunk_readback<T, kE>(dx + r * g.cols + coff, o);
#pragma unroll
          for (int e = 0; e < kE; ++e) acc[e] += o[e];  // sum of dx as stored
        }
      }
    }
  }
  if (part != nullptr) write_col_partials<kE>(acc, sh, part, g, ps);
}

// ---------------------------------------------------------------------------
// bias-dropout-add
// ---------------------------------------------------------------------------

template <typename T, int U, bool HAS_BIAS, bool HAS_RES, bool DROP>
__global__ __launch_bounds__(256) void bias_dropout_add_fwd_kernel(
    const T *__restrict__ x, const T *__restrict__ bias,
    const T *__restrict__ res, T *__restrict__ out,
    uint8_t *__restrict__ mask_out, EltGeom g, DropArgs d) {
  constexpr int kE = io<T>::EPV;
  d = resolve_drop(d);
  const EltPos ps = elt_pos(g);
  if (ps.cc >= g.nchunks) return;
  float b[kE];
  if constexpr (HAS_BIAS) load_chunk<T, kE, false>(bias + (int64_t)ps.cc * kE, b);
  const int64_t coff = (int64_t)ps.cc * kE;
  for (int64_t r0 = ps.slot * g.ty * U + ps.ry; r0 < g.rows;
       r0 += g.slots * g.ty * U) {
    float v[U][kE], rv[U][kE];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = r0 + u * g.ty;
      if (r < g.rows) {
        load_chunk<T, kE>(x + r * g.cols + coff, v[u]);
        if constexpr (HAS_RES) load_chunk<T, kE>(res + r * g.cols + coff, rv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t r = r0 + u * g.ty;
      if (r < g.rows) {
        uint32_t keep = 0xffu;
        if constexpr (DROP)
          keep = chunk_keep_bits<kE>(r, (int)g.cols, ps.cc, d);
        float o[kE];
#pragma unroll
        for (int e = 0; e < kE; ++e) {
          float t = HAS_BIAS ? v[u][e] + b[e] : v[u][e];
          if constexpr (DROP) t = (keep >> e) & 1u ? t * d.scale : 0.f;
          o[e] = HAS_RES ? t + rv[u][e] : t;
        }
        store_chunk<T, kE>(out + r * g.cols + coff, o);
        if (mask_out != nullptr) {
          u32x2 m;
          m.x = m.y = 0;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            m.x |= ((keep >> e) & 1u) << (8 * e);
            if constexpr (kE == 8) m.y |= ((keep >> (4 + e)) & 1u) << (8 * e);
          }
          if constexpr (kE == 8)
            *reinterpret_cast<u32x2 *>(mask_out + r * g.cols + coff) = m;
          else
            *reinterpret_cast<uint32_t *>(mask_out + r * g.cols + coff) = m.x;
        }
      }
    }
  }
}

template <typename T, int U, bool DROP>
__global__ __launch_bounds__(256) void bias_dropout_add_bwd_kernel(
    const T *__restrict__ gr, T *__restrict__ dx, float *__restrict__ part,
    EltGeom g, DropArgs d) {
  constexpr int kE = io<T>::EPV;
  d = resolve_drop(d);
  __shared__ float sh[256 * kE];
  const EltPos ps = elt_pos(g);
  float acc[kE];
#pragma unroll
  for (int e = 0; e < kE; ++e) acc[e] = 0.f;
  if (ps.cc < g.nchunks) {
    const int64_t coff = (int64_t)ps.cc * kE;
    // next step requested before the current one is evaluated, as above
    RawChunk<T, kE> ng[U];
    auto fetch = [&](int64_t r0) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int64_t r = r0 + u * g.ty;
        r = r < g.rows ? r : g.rows - 1;
        ng[u].load(gr + r * g.cols + coff);
      }
    };
    const int64_t step = g.slots * g.ty * U;
    int64_t r0 = ps.slot * g.ty * U + ps.ry;
    if (r0 < g.rows) fetch(r0);
    for (; r0 < g.rows; r0 += step) {
      float gv[U][kE];
#pragma unroll
      for (int u = 0; u < U; ++u) ng[u].unpack(gv[u]);
      if (r0 + step < g.rows) fetch(r0 + step);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t r = r0 + u * g.ty;
        if (r < g.rows) {
          uint32_t keep = 0xffu;
          if constexpr (DROP)
            keep = chunk_keep_bits<kE>(r, (int)g.cols, ps.cc, d);
          float o[kE];
#pragma unroll
          for (int e = 0; e < kE; ++e) {
            float t = gv[u][e];
            if constexpr (DROP) t = (keep >> e) & 1u ? t * d.scale : 0.f;
            o[e] = t;
          }
          store_chunk_readback<T, kE>(dx != nullptr ? dx + r * g.cols + coff : nullptr, o);
#pragma unroll
          for (int e = 0; e < kE; ++e) acc[e] += o[e];  // sum of dx as stored
        }
      }
    }
  }
  if (part != nullptr) write_col_partials<kE>(acc, sh, part, g, ps);
}

// ---------------------------------------------------------------------------
// generic (cols not a multiple of 8, or unaligned pointers): one thread per
// element, grid-stride; the mask is the same function of the element index.
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_fwd_generic_kernel(
    const T *__restrict__ x, const T *__restrict__ bias, T *__restrict__ y,
    int64_t n, int64_t cols) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * 256) {
    float u = io<T>::from_scalar(x[i]);
    if (bias) u += io<T>::from_scalar(bias[i % cols]);
    y[i] = io<T>::to_scalar(gelu_fwd(u));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_bwd_generic_kernel(
    const T *__restrict__ gr, const T *__restrict__ x,
    const T *__restrict__ bias, T *__restrict__ dx, int64_t n, int64_t cols) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * 256) {
    float u = io<T>::from_scalar(x[i]);
    if (bias) u += io<T>::from_scalar(bias[i % cols]);
    dx[i] = io<T>::to_scalar(gelu_bwd(u) * io<T>::from_scalar(gr[i]));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bias_dropout_add_fwd_generic_kernel(
    const T *__restrict__ x, const T *__restrict__ bias,
    const T *__restrict__ res, T *__restrict__ out,
    uint8_t *__restrict__ mask_out, int64_t n, int64_t cols, DropArgs d,
    bool drop) {
  d = resolve_drop(d);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * 256) {
    float t = io<T>::from_scalar(x[i]);
    if (bias) t += io<T>::from_scalar(bias[i % cols]);
    const bool keep = drop ? keep_element(i, d) : true;
    if (drop) t = keep ? t * d.scale : 0.f;
    if (res) t += io<T>::from_scalar(res[i]);
    out[i] = io<T>::to_scalar(t);
    if (mask_out) mask_out[i] = keep ? 1 : 0;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bias_dropout_add_bwd_generic_kernel(
    const T *__restrict__ gr, T *__restrict__ dx, int64_t n, DropArgs d,
    bool drop) {
  d = resolve_drop(d);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * 256) {
    float t = io<T>::from_scalar(gr[i]);
    if (drop) t = keep_element(i, d) ? t * d.scale : 0.f;
    dx[i] = io<T>::to_scalar(t);
  }
}

// dbias alone on the generic path: one thread per column walks the rows and
// sums the values dx would hold, without storing them.
template <typename T>
__global__ __launch_bounds__(256) void bias_dropout_add_dbias_generic_kernel(
    const T *__restrict__ gr, T *__restrict__ dbias, int64_t rows,
    int64_t cols, DropArgs d, bool drop) {
  d = resolve_drop(d);
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= cols) return;
  float s = 0.f;
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t i = r * cols + col;
    float t = io<T>::from_scalar(gr[i]);
    if (drop) t = keep_element(i, d) ? t * d.scale : 0.f;
    s += io<T>::round(t);
  }
  dbias[col] = io<T>::to_scalar(s);
}

// Column sum of an already stored [rows, cols] tensor (generic path only).
template <typename T>
__global__ __launch_bounds__(256) void colsum_generic_kernel(
    const T *__restrict__ a, T *__restrict__ out, int64_t rows, int64_t cols) {
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= cols) return;
  float s = 0.f;
  for (int64_t r = 0; r < rows; ++r) s += io<T>::from_scalar(a[r * cols + col]);
  out[col] = io<T>::to_scalar(s);
}

__global__ __launch_bounds__(256) void philox_mask_kernel(
    uint8_t *__restrict__ mask_out, int64_t n, DropArgs d) {
  d = resolve_drop(d);
  const int64_t ngroups = (n + 7) / 8;
  for (int64_t grp = (int64_t)blockIdx.x * 256 + threadIdx.x; grp < ngroups;
       grp += (int64_t)gridDim.x * 256) {
    const uint32_t keep =
        dropout_keep_bits((uint64_t)grp, d.seed, d.offset, d.threshold);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int64_t i = grp * 8 + e;
      if (i < n) mask_out[i] = (keep >> e) & 1u;
    }
  }
}

__global__ __launch_bounds__(256) void philox_words_kernel(
    uint32_t *__restrict__ out, int64_t ngroups, int64_t first_group,
    uint64_t seed, uint64_t offset) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < ngroups;
       i += (int64_t)gridDim.x * 256) {
    const uint64_t grp = (uint64_t)(first_group + i);
    const Philox4 r = philox4x32_10((uint32_t)offset, (uint32_t)(offset >> 32),
                                    (uint32_t)grp, (uint32_t)(grp >> 32),
                                    (uint32_t)seed, (uint32_t)(seed >> 32));
    out[4 * i + 0] = r.x;
    out[4 * i + 1] = r.y;
    out[4 * i + 2] = r.z;
    out[4 * i + 3] = r.w;
  }
}

// One 128-bit vector per thread, workgroups in memory order: the fastest copy
// measured on MI355X (short-lived waves sweeping one compact window).
__global__ __launch_bounds__(256) void copy_probe_kernel(
    const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t nvec) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec;
       i += stride)
    st16_stream(dst + i, ld16_stream(src + i));
}

__global__ __launch_bounds__(64) void wave_reduce_selftest_kernel(float *out) {
  const int lane = threadIdx.x;
  const float s = wave_sum((float)lane);
  const float m = wave_max((float)((lane * 37) % 64));
  float a = (float)lane, b = (float)(2 * lane);
  a = wave_sum(a);
  b = wave_sum(b);
  if (lane == 17) {
    out[0] = s;
    out[1] = m;
    out[2] = a;
    out[3] = b;
  }
}

// Functor of the generic column sum: the value dx would hold, rounded to the
// storage type, without storing it.
template <typename T> struct DroppedGradient {
  const T *gr;
  int64_t cols;
  DropArgs d;
  bool drop;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float *acc) const {
    const int64_t i = r * cols + c;
    float t = io<T>::from_scalar(gr[i]);
    if (drop) {
      const DropArgs dd = resolve_drop(d);
      t = keep_element(i, dd) ? t * dd.scale : 0.f;
    }
    acc[0] += io<T>::round(t);
  }
};

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
// Column sum of a stored [rows, cols] tensor on the generic path: row slices
// through the workspace when it can be used, else one thread per column.
template <typename T>
static int generic_colsum_of_stored(const void *a, void *out, void *ws,
                                    int64_t ws_bytes, int64_t rows,
                                    int64_t cols, hipStream_t st) {
  const int64_t S = generic_colsum_slices(ws, ws_bytes, 1, rows, cols);
  if (S > 0) {
    StoredValue<T> f{(const T *)a, cols};
    return launch_generic_colsum<1, T>(f, ws, S, rows, cols, out, nullptr, st);
  }
  colsum_generic_kernel<T><<<dim3((unsigned)ceil_div(cols, 256)), 256, 0, st>>>(
      (const T *)a, (T *)out, rows, cols);
  return check_launch("colsum_generic_kernel");
}

static inline int eltwise_unroll(int dflt) {
  const int u = g_tune.eltwise_unroll;
  return u == 1 || u == 2 || u == 4 || (u == 8 && dflt == 8) ? u : dflt;
}

// Tile shape for `cols`: tx lanes wide (a power of two up to 256), ty = 256 /
// tx rows tall.  The widest tile that leaves at most 1/32 of its lanes
// without a chunk is taken (384 chunks -> three tiles of 128 rather than two
// of 256; 8 chunks -> 8 lanes and 32 rows side by side), else the one with the
// fewest idle lanes.
static inline void eltwise_tile(int64_t cols, int E, int *tx, int *ty, int *tiles,
                                int default_max = 256) {
  const int64_t nchunks = ceil_div(cols, E);
  int best = 256;
  int64_t best_waste = -1;
  const int tmax = g_tune.eltwise_tile_max > 0 ? g_tune.eltwise_tile_max : default_max;
  const int tmin = g_tune.eltwise_tile_min > 0 ? g_tune.eltwise_tile_min : 1;
  for (int t = tmax; t >= tmin; t >>= 1) {
    const int64_t waste = ceil_div(nchunks, t) * t - nchunks;
    if (waste * 32 <= nchunks) {
      best = t;
      best_waste = waste;
      break;
    }
    if (best_waste < 0 || waste < best_waste) {
      best = t;
      best_waste = waste;
    }
  }
  *tx = best;
  *ty = 256 / best;
  *tiles = (int)ceil_div(nchunks, best);
}

// Backward: workgroups per column tile = fp32 partial rows.  Measured best on
// MI355X: tiles of at most 128 lanes (two rows side by side in a workgroup)
// and three workgroups per CU, which advance through the rows in step (bf16
// [8192,24576] bias-GeLU backward 223 -> 209 us against 256-lane tiles at two
// per CU; four per CU lose 5 % again); every lane keeps four or eight chunks
// per operand in flight plus the prefetch of the next step, and the partial
// rows stay below one percent of the tensor traffic.
constexpr int kBwdTileMax = 128;
constexpr int kBwdWorkgroupsPerCu = 3;

static int64_t colsum_parts_eltwise_e(int64_t rows, int64_t cols, int E) {
  int tx, ty, tiles;
  eltwise_tile(cols, E, &tx, &ty, &tiles, kBwdTileMax);
  int64_t parts = g_tune.eltwise_rowgroups > 0
                      ? g_tune.eltwise_rowgroups
                      : ((int64_t)device_cu_count() * kBwdWorkgroupsPerCu) / tiles;
  const int64_t min_band =
      g_tune.eltwise_rowgroups > 0 ? ty : (16 > ty ? 16 : ty);
  const int64_t maxp = ceil_div(rows, min_band);
  if (parts > maxp) parts = maxp;
  if (parts < 1) parts = 1;
  return parts;
}

// Upper bound over the chunk widths (the workspace query knows no dtype).
int64_t colsum_parts_eltwise(int64_t rows, int64_t cols) {
  const int64_t a = colsum_parts_eltwise_e(rows, cols, 8);
  const int64_t b = colsum_parts_eltwise_e(rows, cols, 4);
  return a > b ? a : b;
}

static inline EltGeom eltwise_geom_bwd(int64_t rows, int64_t cols, int unroll, int E) {
  EltGeom g;
  g.rows = rows;
  g.cols = cols;
  g.nchunks = (int)(cols / E);
  eltwise_tile(cols, E, &g.tx, &g.ty, &g.tiles, kBwdTileMax);
  const int64_t nsteps = ceil_div(rows, (int64_t)g.ty * unroll);
  g.slots = colsum_parts_eltwise_e(rows, cols, E);
  if (g.slots > nsteps) g.slots = nsteps;
  return g;
}

static inline EltGeom eltwise_geom_fwd(int64_t rows, int64_t cols, int unroll, int E) {
  EltGeom g;
  g.rows = rows;
  g.cols = cols;
  g.nchunks = (int)(cols / E);
  // tiles of at most 128 lanes in the forward kernels as well: two or more rows
  // side by side in a workgroup measure 2-3 % faster than one row of 256 lanes
  // for bias-GeLU at 16384 and 24576 columns (128.5 -> 125 us at [8192, 24576])
  // and the same within 1 % elsewhere
  eltwise_tile(cols, E, &g.tx, &g.ty, &g.tiles, kBwdTileMax);
  const int steps = g_tune.eltwise_fwd_steps > 0 ? g_tune.eltwise_fwd_steps : 1;
  g.slots = ceil_div(ceil_div(rows, (int64_t)g.ty * unroll), steps);
  return g;
}

static inline int64_t flat_grid(int64_t n) {
  int64_t grid = ceil_div(n, 256);
  const int64_t cap = (int64_t)device_cu_count() * 32;
  return grid < cap ? (grid < 1 ? 1 : grid) : cap;
}


#define OSLO_ELT_U(U_, ...)  \
  do {                       \
    switch (U_) {            \
      case 1: { constexpr int U = 1; __VA_ARGS__; } break; \
      case 2: { constexpr int U = 2; __VA_ARGS__; } break; \
      default: { constexpr int U = 4; __VA_ARGS__; } break; \
    }                        \
  } while (0)

// (the forward of bias-dropout-add: one or two steps in flight)
#define OSLO_ELT_U2(U_, ...)  \
  do {                        \
    switch (U_) {             \
      case 1: { constexpr int U = 1; __VA_ARGS__; } break; \
      default: { constexpr int U = 2; __VA_ARGS__; } break; \
    }                         \
  } while (0)

#define OSLO_ELT_U8(U_, ...)  \
  do {                        \
    switch (U_) {             \
      case 1: { constexpr int U = 1; __VA_ARGS__; } break; \
      case 2: { constexpr int U = 2; __VA_ARGS__; } break; \
      case 4: { constexpr int U = 4; __VA_ARGS__; } break; \
      default: { constexpr int U = 8; __VA_ARGS__; } break; \
    }                         \
  } while (0)

template <typename T>
static int run_bias_gelu_fwd(const void *x, const void *bias, void *y,
                             int64_t rows, int64_t cols, hipStream_t st) {
  constexpr int kE = io<T>::EPV;
  const bool vec_ok = cols % kE == 0 && cols <= 0x7fffffff && aligned16(x) && aligned16(y) &&
                      aligned16(bias) && cols / kE <= 0x7fffffff;
  if (!vec_ok) {
    const int64_t n = rows * cols;
    bias_gelu_fwd_generic_kernel<T><<<dim3((unsigned)flat_grid(n)), 256, 0, st>>>(
        (const T *)x, (const T *)bias, (T *)y, n, cols);
    return check_launch("bias_gelu_fwd_generic_kernel");
  }
  const int unroll = eltwise_unroll(2);
  EltGeom g = eltwise_geom_fwd(rows, cols, unroll, kE);
  const int64_t nblocks = g.slots * g.tiles;
  const int64_t per_launch = max_workgroups(256);
  for (g.blk0 = 0; g.blk0 < nblocks; g.blk0 += per_launch) {
    const dim3 grid((unsigned)(nblocks - g.blk0 < per_launch ? nblocks - g.blk0 : per_launch));
    OSLO_ELT_U(unroll, {
      if (bias)
        bias_gelu_fwd_kernel<T, U, true><<<grid, 256, 0, st>>>(
            (const T *)x, (const T *)bias, (T *)y, g);
      else
        bias_gelu_fwd_kernel<T, U, false><<<grid, 256, 0, st>>>(
            (const T *)x, nullptr, (T *)y, g);
    });
    const int rc = check_launch("bias_gelu_fwd_kernel");
    if (rc != OSLO_OK) return rc;
  }
  return OSLO_OK;
}

template <typename T>
static int run_bias_gelu_bwd(const void *gr, const void *x, const void *bias,
                             void *dx, void *dbias, void *ws, int64_t ws_bytes,
                             int64_t rows, int64_t cols, hipStream_t st) {
  constexpr int kE = io<T>::EPV;
  const bool vec_ok = cols % kE == 0 && cols <= 0x7fffffff && aligned16(x) && aligned16(gr) &&
                      aligned16(dx) && aligned16(bias) && aligned16(ws) &&
                      cols / kE <= 0x7fffffff;
  if (!vec_ok) {
    const int64_t n = rows * cols;
    bias_gelu_bwd_generic_kernel<T><<<dim3((unsigned)flat_grid(n)), 256, 0, st>>>(
        (const T *)gr, (const T *)x, (const T *)bias, (T *)dx, n, cols);
    int rc = check_launch("bias_gelu_bwd_generic_kernel");
    if (rc != OSLO_OK || dbias == nullptr) return rc;
    return generic_colsum_of_stored<T>(dx, dbias, ws, ws_bytes, rows, cols, st);
  }
  // eight chunks of each operand in flight per lane (16-bit types; measured
  // 1-3 % faster than four), four for fp32
  const int unroll = eltwise_unroll(sizeof(T) == 2 ? 8 : 4);
  const EltGeom g = eltwise_geom_bwd(rows, cols, unroll, kE);
  const int64_t parts = g.slots;
  const int64_t nblocks = parts * g.tiles;
  OSLO_REQUIRE(nblocks <= max_workgroups(256), "bias_gelu bwd: too many workgroups");
  const dim3 grid((unsigned)nblocks);
  float *part = nullptr;
  if (dbias != nullptr) {
    const int64_t need = parts * cols * (int64_t)sizeof(float);
    if (ws == nullptr || ws_bytes < need)
      return fail(OSLO_ERR_WORKSPACE,
                  "bias_gelu bwd: workspace of %lld bytes needed, %lld given",
                  (long long)need, (long long)ws_bytes);
    part = (float *)ws;
  }
  OSLO_ELT_U8(unroll, {
    // (eight steps in flight are built for the 16-bit types, whose default it is)
    if constexpr (U < 8 || sizeof(T) == 2) {
      if (bias)
        bias_gelu_bwd_kernel<T, U, true><<<grid, 256, 0, st>>>(
            (const T *)gr, (const T *)x, (const T *)bias, (T *)dx, part, g);
      else
        bias_gelu_bwd_kernel<T, U, false><<<grid, 256, 0, st>>>(
            (const T *)gr, (const T *)x, nullptr, (T *)dx, part, g);
    } else {
      return fail(OSLO_ERR_UNSUPPORTED, "bias_gelu bwd: no kernel for %d steps in flight in float32", U);
    }
  });
  int rc = check_launch("bias_gelu_bwd_kernel");
  if (rc != OSLO_OK || dbias == nullptr) return rc;
  if (g_tune.colsum_defer) return rc;  // measurement only: see oslo_colsum_finalize_probe
  return launch_colsum_finalize<T>(part, parts, cols, dbias, nullptr, st);
}

template <typename T>
static int run_bda_fwd(const void *x, const void *bias, const void *res,
                       void *out, uint8_t *mask_out, int64_t rows, int64_t cols,
                       float p, uint64_t seed, uint64_t offset,
                       hipStream_t st) {
  const DropArgs d = make_drop(p, seed, offset);
  const bool drop = p > 0.f;
  constexpr int kE = io<T>::EPV;
  const bool vec_ok = cols % kE == 0 && cols <= 0x7fffffff && aligned16(x) && aligned16(out) &&
                      aligned16(bias) && aligned16(res) &&
                      (reinterpret_cast<uintptr_t>(mask_out) & 7u) == 0 &&
                      cols / kE <= 0x7fffffff;
  if (!vec_ok) {
    const int64_t n = rows * cols;
    bias_dropout_add_fwd_generic_kernel<T>
        <<<dim3((unsigned)flat_grid(n)), 256, 0, st>>>(
            (const T *)x, (const T *)bias, (const T *)res, (T *)out, mask_out,
            n, cols, d, drop);
    return check_launch("bias_dropout_add_fwd_generic_kernel");
  }
  const int unroll = eltwise_unroll(2) > 2 ? 2 : eltwise_unroll(2);
  EltGeom g = eltwise_geom_fwd(rows, cols, unroll, kE);
  const int64_t nblocks = g.slots * g.tiles;
  const int64_t per_launch = max_workgroups(256);
#define OSLO_BDA_FWD(HB, HR, DR)                                            \
  bias_dropout_add_fwd_kernel<T, U, HB, HR, DR><<<grid, 256, 0, st>>>(      \
      (const T *)x, (const T *)bias, (const T *)res, (T *)out, mask_out, g, d)
  for (g.blk0 = 0; g.blk0 < nblocks; g.blk0 += per_launch) {
    const dim3 grid((unsigned)(nblocks - g.blk0 < per_launch ? nblocks - g.blk0 : per_launch));
    OSLO_ELT_U2(unroll, {
      const int key = (bias ? 4 : 0) | (res ? 2 : 0) | (drop ? 1 : 0);
      switch (key) {
        case 0: OSLO_BDA_FWD(false, false, false); break;
        case 1: OSLO_BDA_FWD(false, false, true); break;
        case 2: OSLO_BDA_FWD(false, true, false); break;
        case 3: OSLO_BDA_FWD(false, true, true); break;
        case 4: OSLO_BDA_FWD(true, false, false); break;
        case 5: OSLO_BDA_FWD(true, false, true); break;
        case 6: OSLO_BDA_FWD(true, true, false); break;
        default: OSLO_BDA_FWD(true, true, true); break;
      }
    });
    const int rc = check_launch("bias_dropout_add_fwd_kernel");
    if (rc != OSLO_OK) return rc;
  }
#undef OSLO_BDA_FWD
  return OSLO_OK;
}

template <typename T>
static int run_bda_bwd(const void *gr, void *dx, void *dbias, void *ws,
                       int64_t ws_bytes, int64_t rows, int64_t cols, float p,
                       uint64_t seed, uint64_t offset, hipStream_t st) {
  const DropArgs d = make_drop(p, seed, offset);
  const bool drop = p > 0.f;
  constexpr int kE = io<T>::EPV;
  const bool vec_ok = cols % kE == 0 && cols <= 0x7fffffff && aligned16(gr) && aligned16(dx) &&
                      aligned16(ws) && cols / kE <= 0x7fffffff;
  if (!vec_ok) {
    if (dx == nullptr) {
      const int64_t S = generic_colsum_slices(ws, ws_bytes, 1, rows, cols);
      if (S > 0) {
        DroppedGradient<T> f{(const T *)gr, cols, d, drop};
        return launch_generic_colsum<1, T>(f, ws, S, rows, cols, dbias, nullptr, st);
      }
      bias_dropout_add_dbias_generic_kernel<T>
          <<<dim3((unsigned)ceil_div(cols, 256)), 256, 0, st>>>(
              (const T *)gr, (T *)dbias, rows, cols, d, drop);
      return check_launch("bias_dropout_add_dbias_generic_kernel");
    }
    const int64_t n = rows * cols;
    bias_dropout_add_bwd_generic_kernel<T>
        <<<dim3((unsigned)flat_grid(n)), 256, 0, st>>>((const T *)gr, (T *)dx,
                                                       n, d, drop);
    int rc = check_launch("bias_dropout_add_bwd_generic_kernel");
    if (rc != OSLO_OK || dbias == nullptr) return rc;
    return generic_colsum_of_stored<T>(dx, dbias, ws, ws_bytes, rows, cols, st);
  }
  const int unroll = eltwise_unroll(4);
  const EltGeom g = eltwise_geom_bwd(rows, cols, unroll, kE);
  const int64_t parts = g.slots;
  const int64_t nblocks = parts * g.tiles;
  OSLO_REQUIRE(nblocks <= max_workgroups(256), "bias_dropout_add bwd: too many workgroups");
  const dim3 grid((unsigned)nblocks);
  float *part = nullptr;
  if (dbias != nullptr) {
    const int64_t need = parts * cols * (int64_t)sizeof(float);
    if (ws == nullptr || ws_bytes < need)
      return fail(OSLO_ERR_WORKSPACE,
                  "bias_dropout_add bwd: workspace of %lld bytes needed, %lld "
                  "given",
                  (long long)need, (long long)ws_bytes);
    part = (float *)ws;
  }
  OSLO_ELT_U(unroll, {
    if (drop)
      bias_dropout_add_bwd_kernel<T, U, true><<<grid, 256, 0, st>>>(
          (const T *)gr, (T *)dx, part, g, d);
    else
      bias_dropout_add_bwd_kernel<T, U, false><<<grid, 256, 0, st>>>(
          (const T *)gr, (T *)dx, part, g, d);
  });
  int rc = check_launch("bias_dropout_add_bwd_kernel");
  if (rc != OSLO_OK || dbias == nullptr) return rc;
  if (g_tune.colsum_defer) return rc;  // measurement only: see oslo_colsum_finalize_probe
  return launch_colsum_finalize<T>(part, parts, cols, dbias, nullptr, st);
}

#define OSLO_ELT_DISPATCH(dtype, FN, ...)                      \
  do {                                                         \
    if (dtype == OSLO_DTYPE_F32) return FN<float>(__VA_ARGS__); \
    if (dtype == OSLO_DTYPE_F16) return FN<_Float16>(__VA_ARGS__); \
    return FN<__bf16>(__VA_ARGS__);                            \
  } while (0)

static int check_elt(const char *what, int64_t rows, int64_t cols, int dtype) {
  if (!valid_dtype(dtype))
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: unknown dtype %d", what, dtype);
  if (rows < 0 || cols < 1)
    return fail(OSLO_ERR_INVALID_ARGUMENT, "%s: bad shape [%lld, %lld]", what,
                (long long)rows, (long long)cols);
  return OSLO_OK;
}

// Zero parameter gradient for an empty batch (P = 0 partial rows).
template <typename T>
static int zero_vector(void *out, int64_t cols, hipStream_t st) {
  return launch_colsum_finalize<T>(nullptr, 0, cols, out, nullptr, st);
}

}  // namespace oslo

extern "C" {

using namespace oslo;

int oslo_bias_gelu_fwd(const void *x, const void *bias, void *y, int64_t rows,
                       int64_t cols, int dtype, void *stream) {
  oslo::tune_snapshot();
  int rc = check_elt("bias_gelu fwd", rows, cols, dtype);
  if (rc != OSLO_OK) return rc;
  if (rows == 0) return OSLO_OK;
  OSLO_REQUIRE(x && y, "bias_gelu fwd: null tensor pointer");
  OSLO_ELT_DISPATCH(dtype, run_bias_gelu_fwd, x, bias, y, rows, cols,
                    (hipStream_t)stream);
}

int oslo_bias_gelu_bwd(const void *g, const void *x, const void *bias,
                       void *dx, void *dbias, void *workspace,
                       int64_t workspace_bytes, int64_t rows, int64_t cols,
                       int dtype, void *stream) {
  oslo::tune_snapshot();
  int rc = check_elt("bias_gelu bwd", rows, cols, dtype);
  if (rc != OSLO_OK) return rc;
  if (rows == 0) {
    if (dbias) OSLO_ELT_DISPATCH(dtype, zero_vector, dbias, cols, (hipStream_t)stream);
    return OSLO_OK;
  }
  OSLO_REQUIRE(g && x && dx, "bias_gelu bwd: null tensor pointer");
  OSLO_ELT_DISPATCH(dtype, run_bias_gelu_bwd, g, x, bias, dx, dbias, workspace,
                    workspace_bytes, rows, cols, (hipStream_t)stream);
}

int oslo_bias_dropout_add_fwd(const void *x, const void *bias,
                              const void *residual, void *out,
                              uint8_t *mask_out, int64_t rows, int64_t cols,
                              float p, uint64_t seed, uint64_t offset,
                              int dtype, void *stream) {
  oslo::tune_snapshot();
  int rc = check_elt("bias_dropout_add fwd", rows, cols, dtype);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(p >= 0.f && p <= 1.f, "bias_dropout_add fwd: p = %f not in [0, 1]",
               (double)p);
  if (rows == 0) return OSLO_OK;
  OSLO_REQUIRE(x && out, "bias_dropout_add fwd: null tensor pointer");
  OSLO_ELT_DISPATCH(dtype, run_bda_fwd, x, bias, residual, out, mask_out, rows,
                    cols, p, seed, offset, (hipStream_t)stream);
}

int oslo_bias_dropout_add_bwd(const void *g, void *dx, void *dbias,
                              void *workspace, int64_t workspace_bytes,
                              int64_t rows, int64_t cols, float p,
                              uint64_t seed, uint64_t offset, int dtype,
                              void *stream) {
  oslo::tune_snapshot();
  int rc = check_elt("bias_dropout_add bwd", rows, cols, dtype);
  if (rc != OSLO_OK) return rc;
  OSLO_REQUIRE(p >= 0.f && p <= 1.f, "bias_dropout_add bwd: p = %f not in [0, 1]",
               (double)p);
  if (rows == 0) {
    if (dbias) OSLO_ELT_DISPATCH(dtype, zero_vector, dbias, cols, (hipStream_t)stream);
    return OSLO_OK;
  }
  OSLO_REQUIRE(g != nullptr, "bias_dropout_add bwd: null gradient pointer");
  OSLO_REQUIRE(dx != nullptr || dbias != nullptr,
               "bias_dropout_add bwd: nothing to compute");
  OSLO_ELT_DISPATCH(dtype, run_bda_bwd, g, dx, dbias, workspace,
                    workspace_bytes, rows, cols, p, seed, offset,
                    (hipStream_t)stream);
}

int oslo_philox_mask(uint8_t *mask_out, int64_t n, float p, uint64_t seed,
                     uint64_t offset, void *stream) {
  oslo::tune_snapshot();
  OSLO_REQUIRE(n >= 0 && p >= 0.f && p <= 1.f, "philox_mask: bad arguments");
  if (n == 0) return OSLO_OK;
  OSLO_REQUIRE(mask_out != nullptr, "philox_mask: null output");
  philox_mask_kernel<<<dim3((unsigned)flat_grid((n + 7) / 8)), 256, 0,
                       (hipStream_t)stream>>>(mask_out, n,
                                              make_drop(p, seed, offset));
  return check_launch("philox_mask_kernel");
}

int oslo_philox_words(uint32_t *out, int64_t ngroups, int64_t first_group,
                      uint64_t seed, uint64_t offset, void *stream) {
  oslo::tune_snapshot();
  OSLO_REQUIRE(ngroups >= 0, "philox_words: bad arguments");
  if (ngroups == 0) return OSLO_OK;
  OSLO_REQUIRE(out != nullptr, "philox_words: null output");
  philox_words_kernel<<<dim3((unsigned)flat_grid(ngroups)), 256, 0,
                        (hipStream_t)stream>>>(out, ngroups, first_group, seed,
                                               offset);
  return check_launch("philox_words_kernel");
}

int oslo_colsum_finalize_probe(const void *partial_rows, int64_t parts, int64_t cols,
                               void *out0, void *out1, void *out2, int dtype,
                               void *stream) {
  oslo::tune_snapshot();
  if (!valid_dtype(dtype) || parts < 0 || cols < 4 || cols % 4 != 0 || !partial_rows || !out0)
    return fail(OSLO_ERR_INVALID_ARGUMENT, "colsum_finalize_probe: bad arguments");
  const int na = out2 ? 3 : (out1 ? 2 : 1);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == OSLO_DTYPE_F32)
    return launch_colsum_finalize<float>((const float *)partial_rows, parts, cols, out0, out1, st, out2, na);
  if (dtype == OSLO_DTYPE_F16)
    return launch_colsum_finalize<_Float16>((const float *)partial_rows, parts, cols, out0, out1, st, out2, na);
  return launch_colsum_finalize<__bf16>((const float *)partial_rows, parts, cols, out0, out1, st, out2, na);
}

int oslo_copy_probe(const void *src, void *dst, int64_t bytes, void *stream) {
  oslo::tune_snapshot();
  OSLO_REQUIRE(bytes >= 0 && bytes % 16 == 0 && aligned16(src) && aligned16(dst),
               "copy_probe: bytes must be a multiple of 16 and pointers "
               "16-byte aligned");
  if (bytes == 0) return OSLO_OK;
  const int64_t nvec = bytes / 16;
  int64_t grid = ceil_div(nvec, 256);
  if (grid > max_workgroups(256)) grid = max_workgroups(256);  // (the kernel strides over the vectors)
  copy_probe_kernel<<<dim3((unsigned)grid), 256, 0, (hipStream_t)stream>>>(
      (const u32x4 *)src, (u32x4 *)dst, nvec);
  return check_launch("copy_probe_kernel");
}

int oslo_wave_reduce_selftest(float *out4, void *stream) {
  oslo::tune_snapshot();
  OSLO_REQUIRE(out4 != nullptr, "wave_reduce_selftest: null output");
  wave_reduce_selftest_kernel<<<1, 64, 0, (hipStream_t)stream>>>(out4);
  return check_launch("wave_reduce_selftest_kernel");
}

}  // extern "C"
