// Scaled causal (upper-triangular) and padding-masked softmax, forward and
// backward, for gfx950.
//
// A row of sk keys is held in registers by `wpr` wavefronts (one wavefront
// for sk <= 64 * VPL * E); a wavefront processes RPW rows at once so that
// short rows still keep several 128-bit loads in flight per lane, and rows of
// at most 32 chunks (256 16-bit keys) lie side by side in a wavefront, 8, 16
// or 32 lanes each, so that no lane idles.  Keys that
// are masked out are never loaded: the causal kernels stop at the diagonal,
// the masked kernels read the mask bytes of a chunk first and skip the chunk
// when all of them are set.  Probabilities of masked keys are written as
// exact zeros.
//
// Semantics: oslo/transformers/models/gpt2/modeling_gpt2.py:116-138 (causal),
// oslo/transformers/models/bert/modeling_bert.py:298-306 (additive padding
// mask); entry-point shapes follow
// oslo/torch/_C/csrc/FusedScaleMaskSoftmaxBinder.cpp:39-105.
#pragma once
#include "capi.h"
#include "common.hip.h"

namespace oslo {

constexpr int kModeCausal = 0;
constexpr int kModeMasked = 1;
constexpr int kModeDense = 2;  // backward without a mask
constexpr int kModeBias = 3;   // additive floating-point term instead of a mask

// An additive term at or below this value (the lowest finite bfloat16; the
// lowest finite float and -inf lie below it) absorbs any logit it is added to:
// the sum is the term itself in float arithmetic, so the logit need not be read.
constexpr float kBiasHidden = -3.38e38f;

constexpr float kLog2e = 1.4426950408889634f;

struct SoftmaxGeom {
  int64_t rows;     // total softmax rows
  int sq, sk;
  int np;           // heads (masked mode)
  int mask_b_stride_rows;  // mask rows per batch entry: mask_sq, or 0 if mask_b == 1
  int mask_per_query;      // 1 if mask_sq == sq else 0
  int wpr, rpb;     // waves per row, rows per workgroup pass (without RPW)
  int causal;       // masked mode: key j of query i is also hidden when j > i + (sk - sq)
  // n / sq and n / np for n < 2^31 as mulhi(n, mul) >> shift (shift == 32: divisor 1),
  // filled in by set_fast_div on the host
  uint32_t sq_mul = 0, sq_shift = 32, np_mul = 0, np_shift = 32;
  float inv_sk = 0.f;  // 1 / sk, the value of a row without a visible key
  // index of the launch's first workgroup among those of the whole problem (a
  // problem beyond 2^32 work-items takes several launches)
  int64_t blk0 = 0;
  // additive term (kModeBias): element strides of its batch, head and query
  // dimensions (0 = broadcast), bytes per element, and whether a chunk whose
  // terms are all <= kBiasHidden skips the load of its logits
  int64_t bias_sb = 0, bias_sh = 0, bias_sq = 0;
  int bias_esize = 0, bias_skip = 0;
  // An additive term shared by the batch (a position bias [1, np, sq, sk]): the
  // rows are visited in runs of 2^group_shift consecutive rows of one batch
  // entry, then the same rows of the next entry, so that the nb rows that read
  // one row of the term run close to each other and the L2 serves it to all
  // but the first of them (measured at [16, 16, 1024, 1024] fp16: 221 us in
  // stored order, 203 us with runs of one row, 169 us with runs of 32, which
  // keep the logits in long contiguous pieces).  With xcd_wpx != 0 workgroup w
  // works on block (w % 8) * xcd_wpx + w / 8, which puts consecutive blocks on
  // one of the eight dies (191 us with runs of one row, 179-181 us with runs
  // of 32-128: not the default).
  int batch_inner = 0, nb = 1;
  int group_shift = 0;   // the batch index advances after 2^group_shift rows
  uint32_t nb_mul = 0, nb_shift = 32;
  int64_t hq_rows = 0;   // np * sq
  int64_t xcd_wpx = 0;   // 0: blocks in launch order
  // Order of the queries of one attention matrix under the diagonal: 0 = long
  // rows first, 1 = as stored, 2 = long and short rows in turn (the k-th row
  // visited is sq - 1 - k / 2 for even k and k / 2 for odd k), so that any run
  // of consecutive rows moves the same number of bytes.
  int causal_order = 0;
};

// Query index of the k-th row visited in an attention matrix of sq queries.
__device__ __forceinline__ int causal_query(const SoftmaxGeom &g, int k) {
  if (g.causal_order == 2) return (k & 1) ? (k >> 1) : g.sq - 1 - (k >> 1);
  return g.causal_order == 1 ? k : g.sq - 1 - k;
}

// The block of rows a workgroup works on.
__device__ __forceinline__ int64_t work_block(const SoftmaxGeom &g) {
  if (g.xcd_wpx != 0) return (int64_t)(blockIdx.x & 7u) * g.xcd_wpx + (int64_t)(blockIdx.x >> 3);
  return (int64_t)blockIdx.x + g.blk0;
}

// Division of n < 2^31 by a divisor 1 <= d < 2^31 fixed for the launch: with
// l = ceil(log2 d) and mul = ceil(2^(31 + l) / d) < 2^32, floor(n / d) equals
// mulhi(n, mul) >> (l - 1) exactly (the error term n * e / (d * 2^(31 + l)) with
// e < d stays below 2^-l <= 1 / d).  A run-time division costs about as many
// vector instructions as the softmax of a short row.
static inline void fast_div_make(uint32_t d, uint32_t *mul, uint32_t *shift) {
  if (d <= 1) {
    *mul = 0;
    *shift = 32;
    return;
  }
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;
  *mul = (uint32_t)(((1ull << (31 + l)) + d - 1) / d);
  *shift = l - 1;
}

static inline void set_fast_div(SoftmaxGeom &g) {
  fast_div_make((uint32_t)g.sq, &g.sq_mul, &g.sq_shift);
  fast_div_make((uint32_t)g.np, &g.np_mul, &g.np_shift);
  fast_div_make((uint32_t)g.nb, &g.nb_mul, &g.nb_shift);
  g.inv_sk = 1.0f / (float)g.sk;
  g.causal_order = g_tune.softmax_causal_order > 0 ? g_tune.softmax_causal_order - 1 : 0;
}

__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t mul, uint32_t shift) {
  return shift == 32 ? n : __umulhi(n, mul) >> shift;
}

// 1 / s for the row sum s >= 1 of a softmax: the hardware reciprocal refined by
// one Newton step (within an ulp of the quotient; an IEEE division costs ten
// instructions).  Every softmax kernel forms its normaliser with this function.
__device__ __forceinline__ float row_recip(float s) {
  const float r = __builtin_amdgcn_rcpf(s);
  return __builtin_fmaf(r, __builtin_fmaf(-s, r, 1.0f), r);
}

// Reductions over the wpr (<= 16) consecutive waves of a row: lane 0 of each
// wave publishes its wave's value in LDS, lane l < wpr then reads the value of
// wave first + l and one DPP row reduction combines them.  With LPR < 64 a
// row belongs to LPR consecutive lanes of one wave (wpr == 1) and the
// reduction stays inside that group.
template <int LPR = kWave>
__device__ __forceinline__ float row_reduce_sum(float a, float *red, int wave,
                                                int first, int wpr, int lane) {
  if constexpr (LPR < kWave) return group_allreduce<OpSum, LPR>(a);
  a = wave_sum(a);
  if (wpr > 1) {
    if (lane == 0) red[wave] = a;
    __syncthreads();
    const bool own = lane < wpr;
    const float r = red[own ? first + lane : first];
    a = row16_allreduce<OpSum>(own ? r : 0.f);
  }
  return a;
}
template <int LPR = kWave>
__device__ __forceinline__ float row_reduce_max(float a, float *red, int wave,
                                                int first, int wpr, int lane) {
  if constexpr (LPR < kWave) return group_allreduce<OpMax, LPR>(a);
  a = wave_max(a);
  if (wpr > 1) {
    if (lane == 0) red[wave] = a;
    __syncthreads();
    // lanes >= wpr repeat the first wave's value, which leaves the maximum unchanged
    a = row16_allreduce<OpMax>(red[lane < wpr ? first + lane : first]);
  }
  return a;
}

// Mask bytes of one chunk -> bit e set when key e of the chunk is masked out.
template <int E>
__device__ __forceinline__ uint32_t load_mask_bits(const uint8_t *p) {
  uint32_t bits = 0;
  if constexpr (E == 8) {
    const u32x2 m = *reinterpret_cast<const u32x2 *>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      bits |= ((m.x >> (8 * e)) & 0xffu) ? (1u << e) : 0u;
      bits |= ((m.y >> (8 * e)) & 0xffu) ? (1u << (4 + e)) : 0u;
    }
  } else {
    const uint32_t m = *reinterpret_cast<const uint32_t *>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      bits |= ((m >> (8 * e)) & 0xffu) ? (1u << e) : 0u;
  }
  return bits;
}

// Mask bits of chunk c (E keys) of a row that sees `visible` keys through the
// diagonal: the keys from `visible` on are hidden as well.  Chunks that lie
// beyond the diagonal altogether do not read their mask bytes.
template <int E>
__device__ __forceinline__ uint32_t masked_chunk_bits(const uint8_t *mrow, int c,
                                                      int visible) {
  constexpr uint32_t kAllBits = (1u << E) - 1u;
  const int left = visible - c * E;  // keys of the chunk below the diagonal
  if (left <= 0) return kAllBits;
  uint32_t mb = load_mask_bits<E>(mrow + (int64_t)c * E);
  if (left < E) mb |= kAllBits & ~((1u << left) - 1u);
  return mb;
}

// Row bookkeeping shared by forward and backward.  Rows are numbered so that
// a workgroup's rows are consecutive; under the diagonal the queries of an
// attention matrix are visited in the order causal_query() gives.
template <int MODE>
__device__ __forceinline__ void row_setup(const SoftmaxGeom &g, int64_t r,
                                          const uint8_t *mask, int64_t &row,
                                          int &visible,
                                          const uint8_t *&mrow) {
  mrow = nullptr;
  visible = g.sk;
  row = r;
  // multiplication by a precomputed reciprocal where the row count allows it
  const bool small = g.rows <= 0x7fffffff;
  if constexpr (MODE == kModeCausal) {
    const int64_t batch =
        small ? (int64_t)fast_div((uint32_t)r, g.sq_mul, g.sq_shift) : r / g.sq;
    const int qi = causal_query(g, (int)(r - batch * g.sq));
    row = batch * g.sq + qi;
    int v = qi + 1 + (g.sk - g.sq);
    visible = v < 0 ? 0 : (v > g.sk ? g.sk : v);
  } else if constexpr (MODE == kModeMasked) {
    const int64_t bh =
        small ? (int64_t)fast_div((uint32_t)r, g.sq_mul, g.sq_shift) : r / g.sq;
    int qi = (int)(r - bh * g.sq);
    if (g.causal) {  // uniform over the launch: the order of causal mode
      qi = causal_query(g, qi);
      row = bh * g.sq + qi;
      const int v = qi + 1 + (g.sk - g.sq);
      visible = v < 0 ? 0 : (v > g.sk ? g.sk : v);
    }
    const int64_t bi =
        small ? (int64_t)fast_div((uint32_t)bh, g.np_mul, g.np_shift) : bh / g.np;
    const int64_t mr =
        bi * g.mask_b_stride_rows + (g.mask_per_query ? qi : 0);
    mrow = mask + mr * g.sk;
  } else if constexpr (MODE == kModeBias) {
    if (g.batch_inner) {
      // r = (run * nb + batch entry) * 2^group_shift + row within the run
      const int64_t t = r >> g.group_shift;
      const int64_t in_run = r - (t << g.group_shift);
      const int64_t run =
          small ? (int64_t)fast_div((uint32_t)t, g.nb_mul, g.nb_shift) : t / g.nb;
      r = (t - run * g.nb) * g.hq_rows + (run << g.group_shift) + in_run;
      row = r;
    }
    const int64_t bh =
        small ? (int64_t)fast_div((uint32_t)r, g.sq_mul, g.sq_shift) : r / g.sq;
    int qi = (int)(r - bh * g.sq);
    if (g.causal) {
      qi = causal_query(g, qi);
      row = bh * g.sq + qi;
      const int v = qi + 1 + (g.sk - g.sq);
      visible = v < 0 ? 0 : (v > g.sk ? g.sk : v);
    }
    const int64_t bi =
        small ? (int64_t)fast_div((uint32_t)bh, g.np_mul, g.np_shift) : bh / g.np;
    const int64_t hi = bh - bi * g.np;
    // (mask is the additive term's base address here; null in a backward
    //  pass that does not use it)
    mrow = mask + (bi * g.bias_sb + hi * g.bias_sh + qi * g.bias_sq) * g.bias_esize;
  }
}

// One chunk of the additive term, E values of the logits' type T or of float
// (a launch-uniform choice, so one kernel serves both), converted to float as
// soon as it arrives: the float form is no wider than a float chunk as loaded.
template <typename T, int E>
__device__ __forceinline__ void load_bias_chunk(const uint8_t *row, int c, bool f32, float *f) {
  if (sizeof(T) == 4 || f32) {
#pragma unroll
    for (int v = 0; v < E / 4; ++v)
      io<float>::unpack(ld16_cached(row + ((int64_t)c * E + 4 * v) * 4), f + 4 * v);
  } else {
    io<T>::unpack(ld16_cached(row + (int64_t)c * E * (int64_t)sizeof(T)), f);
  }
}

// The same in two steps, for code that issues all its loads before it
// converts any of them: the chunk as loaded (E / 4 vectors, the first one only
// for a 16-bit term), then its conversion.
template <typename T, int E>
__device__ __forceinline__ void load_bias_raw(const uint8_t *row, int c, bool f32, u32x4 *r) {
  if (sizeof(T) == 4 || f32) {
#pragma unroll
    for (int v = 0; v < E / 4; ++v) r[v] = ld16_cached(row + ((int64_t)c * E + 4 * v) * 4);
  } else {
    r[0] = ld16_cached(row + (int64_t)c * E * (int64_t)sizeof(T));
  }
}
template <typename T, int E>
__device__ __forceinline__ void unpack_bias_raw(const u32x4 *r, bool f32, float *f) {
  if (sizeof(T) == 4 || f32) {
#pragma unroll
    for (int v = 0; v < E / 4; ++v) io<float>::unpack(r[v], f + 4 * v);
  } else {
    io<T>::unpack(r[0], f);
  }
}

// every term of the chunk absorbs its logit
template <int E>
__device__ __forceinline__ bool bias_all_hidden(const float *f) {
  float m = f[0];
#pragma unroll
  for (int e = 1; e + 1 < E; e += 2) m = fmaxf(fmaxf(m, f[e]), f[e + 1]);  // v_max3_f32
  if constexpr (E % 2 == 0) m = fmaxf(m, f[E - 1]);
  return m <= kBiasHidden;  // (false for NaN)
}

// scalar read of element i of an additive-term row (generic kernels)
template <typename T>
__device__ __forceinline__ float bias_at(const uint8_t *row, int i, bool f32) {
  if (sizeof(T) == 4 || f32) return reinterpret_cast<const float *>(row)[i];
  return io<T>::from_scalar(reinterpret_cast<const T *>(row)[i]);
}

// DROP: dropout is applied to the probabilities before they are written
// (oslo/transformers/models/gpt2/modeling_gpt2.py:138-142,
// oslo/transformers/models/bert/modeling_bert.py:306-310) and the row
// statistics {max of the log2-domain logits, 1 / sum} go to stats[row], from
// which the backward pass recomputes the probabilities.  A row without a
// visible key stores {0, -1 / sk}.
//
// LPR lanes hold a row: 64 (a row takes whole waves), or 8 / 16 / 32 for rows
// of at most LPR chunks, where a wave works on 64 / LPR rows side by side
// (then VPL == 1 and wpr == 1).
template <typename T, int VPL, int RPW, int MODE, bool DROP, int LPR = kWave>
__global__ __launch_bounds__(1024) void softmax_fwd_kernel(
    const T *__restrict__ x, const uint8_t *__restrict__ mask,
    T *__restrict__ y, float *__restrict__ stats, SoftmaxGeom g, float scale,
    DropArgs d) {
  d = resolve_drop(d);
  constexpr int E = io<T>::EPV;
  constexpr uint32_t kAll = (1u << E) - 1u;
  __shared__ float red[2][16];
  const int lane = threadIdx.x & 63;
  // the wave index is uniform: keep it (and the row arithmetic) in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rslot = g.wpr == 1 ? wave : wave / g.wpr;  // (uniform: the division is skipped)
  const int first = rslot * g.wpr;
  const int nchunks = g.sk / E;
  const int cstride = LPR == kWave ? kWave * g.wpr : LPR;
  constexpr int SUB = kWave / LPR;  // rows side by side in a wave
  const int sl = LPR == kWave ? lane : (lane & (LPR - 1));
  const int c0 = (wave - first) * kWave + sl;
  const float ninf = -__builtin_inff();

  // first row of this lane: the wave's first row plus the lane group's index
  const int64_t rbase =
      (work_block(g) * g.rpb + rslot) * (RPW * SUB) +
      (LPR == kWave ? 0 : lane / LPR);

  float v[RPW][VPL][E];
  uint32_t mbits[RPW][VPL];  // bit e set: key masked out
  int64_t row[RPW];
  bool rvalid[RPW];
  // additive term: a query that the diagonal leaves without any key (sq > sk)
  // gets zeros (its neighbours in the wave may well see keys, so the
  // wave-uniform shortcuts below do not catch it)
  bool nokey[RPW];
  const uint8_t *mrow0 = nullptr;
  // additive term (kModeBias): the chunks as loaded, and whether a chunk's
  // logits were left unread
  constexpr bool kBias = MODE == kModeBias;
  float bv[kBias ? RPW : 1][kBias ? VPL : 1][kBias ? E : 1];
  u32x4 braw[kBias ? RPW : 1][kBias ? VPL : 1][kBias ? E / 4 : 1];
  RawChunk<T, E> xraw[kBias ? RPW : 1][kBias ? VPL : 1];
  bool bhid[kBias ? RPW : 1][kBias ? VPL : 1];
  const bool bias_f32 = g.bias_esize == 4;

#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int64_t r = rbase + j * SUB;
    rvalid[j] = r < g.rows;
    int visible = 0;
    const uint8_t *mrow = nullptr;
    row[j] = 0;
    if (rvalid[j]) row_setup<MODE>(g, r, mask, row[j], visible, mrow);
    nokey[j] = MODE == kModeBias && rvalid[j] && visible <= 0;
    // consecutive rows of a wave normally share their mask row (a key-padding
    // mask [b, 1, 1, sk]): its bits are then read and unpacked once
    bool shared = false;
    if constexpr (MODE == kModeMasked && RPW > 1) {
      if (j == 0) mrow0 = mrow;
      shared = j > 0 && rvalid[j] && rvalid[0] && mrow == mrow0 && !g.causal;
    }
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      uint32_t mb = (1u << E) - 1u;
      if (shared) {
        mb = mbits[0][k];
      } else if (rvalid[j] && c < nchunks) {
        if constexpr (MODE == kModeCausal || MODE == kModeBias) {
          // (visible == sk without a diagonal)
          const int left = visible - c * E;  // visible keys in this chunk
          mb = left >= E ? 0u : (left <= 0 ? mb : (mb & ~((1u << left) - 1u)));
        } else {
          mb = masked_chunk_bits<E>(mrow, c, visible);
        }
      }
      mbits[j][k] = mb;
      if constexpr (MODE == kModeBias) {
        // the additive term of every chunk that has a key below the diagonal
        // (cached loads: its rows are normally shared by many rows of logits)
        // (all of them requested before any is converted: a conversion
        //  waits for its load)
        bhid[j][k] = false;
        if (mb != kAll) load_bias_raw<T, E>(mrow, c, bias_f32, braw[j][k]);
      }
    }
  }
  if constexpr (MODE == kModeBias) {
    // a chunk whose terms all absorb their logits takes the terms as its
    // sums: the logits are not read
    if (g.bias_skip) {
#pragma unroll
      for (int j = 0; j < RPW; ++j)
#pragma unroll
        for (int k = 0; k < VPL; ++k)
          if (mbits[j][k] != kAll) {
            unpack_bias_raw<T, E>(braw[j][k], bias_f32, bv[j][k]);
            bhid[j][k] = bias_all_hidden<E>(bv[j][k]);
          }
    }
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const T *xr = x + row[j] * g.sk;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      // (a chunk without a visible key is not loaded; its registers are never
      //  used: every select below takes the masked branch for it)
      bool want = mbits[j][k] != (1u << E) - 1u;
      if constexpr (MODE == kModeBias) {
        if (want && !bhid[j][k]) xraw[j][k].load(xr + (int64_t)c * E);
      } else {
        if (want) load_chunk<T, E>(xr + (int64_t)c * E, v[j][k]);
      }
    }
  }
  if constexpr (MODE == kModeBias) {
    // (without the test above the logits were requested together with the
    //  terms: the terms are converted only now)
    if (!g.bias_skip) {
#pragma unroll
      for (int j = 0; j < RPW; ++j)
#pragma unroll
        for (int k = 0; k < VPL; ++k)
          if (mbits[j][k] != kAll) unpack_bias_raw<T, E>(braw[j][k], bias_f32, bv[j][k]);
    }
#pragma unroll
    for (int j = 0; j < RPW; ++j)
#pragma unroll
      for (int k = 0; k < VPL; ++k)
        if (mbits[j][k] != kAll && !bhid[j][k]) xraw[j][k].unpack(v[j][k]);
  }

  // Wave-uniform shortcuts: where no lane of the wave sees a key of chunk
  // slot (j, k) the arithmetic is skipped altogether; where every lane sees
  // all its keys the per-element mask selects are skipped.  The logits are
  // kept in the log2 domain, t = x * (scale * log2 e), so exp is one exp2.
  bool none_visible[RPW][VPL], all_visible[RPW][VPL];
  // additive term: no lane of the wave read the logits of the slot (every
  // chunk of it lies beyond the diagonal or under terms that absorb it)
  bool slot_unread[kBias ? RPW : 1][kBias ? VPL : 1];
#pragma unroll
  for (int j = 0; j < RPW; ++j)
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      none_visible[j][k] = __builtin_amdgcn_ballot_w64(mbits[j][k] != kAll) == 0;
      all_visible[j][k] = __builtin_amdgcn_ballot_w64(mbits[j][k] != 0u) == 0;
      if constexpr (kBias)
        slot_unread[j][k] =
            __builtin_amdgcn_ballot_w64(mbits[j][k] != kAll && !bhid[j][k]) == 0;
    }
  const float c2 = scale * kLog2e;

  float mx[RPW];
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    float m = ninf;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      if (none_visible[j][k]) continue;
      if constexpr (MODE == kModeBias) {
        // the sum scale * x + term as one fused multiply-add, kept in the
        // natural domain: a large negative term (-10000) then costs the logit
        // one rounding, as in a float evaluation of the unfused chain
        const float *bf = bv[j][k];
        // (wave-uniform: no lane of the wave left the logits of this slot unread)
        const bool no_skip = __builtin_amdgcn_ballot_w64(bhid[j][k]) == 0;
        if (DROP && no_skip && all_visible[j][k]) {
          // (the common slot as a branch of its own, two instructions a key, in
          //  the kernels with dropout, which are bound by instruction issue:
          //  204 -> 186 us at [16, 16, 1024, 1024] fp16; the kernels without
          //  dropout are bound by memory there and measure 2 % slower with
          //  the branch, 163 -> 167 us)
#pragma unroll
          for (int e = 0; e < E; ++e) {
            const float t = __builtin_fmaf(v[j][k][e], scale, bf[e]);
            v[j][k][e] = t;
            m = fmaxf(m, t);
          }
        } else {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            float t = bhid[j][k] ? bf[e] : __builtin_fmaf(v[j][k][e], scale, bf[e]);
            t = (mbits[j][k] >> e) & 1u ? ninf : t;
            v[j][k][e] = t;
            m = fmaxf(m, t);
          }
        }
        continue;
      }
      if (all_visible[j][k]) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          // (rounded product, never fused into the later subtraction: the
          //  backward pass of the dropout variant recomputes it bit for bit)
          const float t = mul_rn(v[j][k][e], c2);
          v[j][k][e] = t;
          m = fmaxf(m, t);
        }
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const float t = (mbits[j][k] >> e) & 1u ? ninf : mul_rn(v[j][k][e], c2);
          v[j][k][e] = t;
          m = fmaxf(m, t);
        }
      }
    }
    mx[j] = m;
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j)
    mx[j] = row_reduce_max<LPR>(mx[j], red[0], wave, first, g.wpr, lane);
  // (one barrier separates the two LDS areas; RPW > 1 implies wpr == 1,
  //  where LDS is not used at all)

  float sm[RPW];
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    float s = 0.f;
    // (with an additive term a row of -inf sums is NaN, as torch.softmax
    //  returns it: the maximum is subtracted as it is)
    const float off = (mx[j] == ninf && !kBias) || nokey[j] ? 0.f : mx[j];
    // (additive term: a slot whose logits were all left unread holds exact
    //  zeros as soon as every row of the wave has another key: no exponentials)
    if constexpr (kBias) {
      const bool hidden_are_zero = __builtin_amdgcn_ballot_w64(!(mx[j] > kBiasHidden)) == 0;
      // (such a slot is written as zeros below, like one that no lane sees:
      //  its registers are not touched again)
#pragma unroll
      for (int k = 0; k < VPL; ++k)
        if (slot_unread[j][k] && hidden_are_zero) none_visible[j][k] = true;
    }
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      if (none_visible[j][k]) continue;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        float d = sub_rn(v[j][k][e], off);
        if constexpr (kBias) d = mul_rn(d, kLog2e);
        const float p = __builtin_amdgcn_exp2f(d);
        v[j][k][e] = p;  // exp2(-inf) == 0 for masked keys
        s += p;
      }
    }
    sm[j] = s;
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j)
    sm[j] = row_reduce_sum<LPR>(sm[j], red[1], wave, first, g.wpr, lane);

#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    if (!rvalid[j]) continue;
    // a row without any visible key: uniform distribution, as softmax of a
    // constant fill value gives
    const bool empty = mx[j] == ninf && !kBias;
    const float inv = empty || nokey[j] ? 0.f : row_recip(sm[j]);
    const float fill = empty ? g.inv_sk : 0.f;
    T *yr = y + row[j] * g.sk;
    if constexpr (DROP) {
      if (c0 == 0) {
        stats[2 * row[j]] = empty || nokey[j] ? 0.f : mx[j];
        stats[2 * row[j] + 1] = empty ? -fill : inv;
      }
    }
    // A 4-element chunk is half a dropout group, and the lanes 2i and 2i + 1
    // hold the two halves: instead of evaluating every group twice, the even
    // lane draws the pair's group of chunk slot 2m, the odd lane that of slot
    // 2m + 1, and one DPP swap hands each lane the other's result.  (Rows of a
    // multiple of 8 keys, so that groups do not straddle rows; the row and the
    // conditions below are uniform over the wave, so all lanes are active.)
    constexpr bool kPairDraw = DROP && E == 4 && LPR == kWave && VPL % 2 == 0;
    uint32_t keepk[kPairDraw ? VPL : 1];
    bool paired = false;
    if constexpr (kPairDraw) {
      if ((g.sk & 7) == 0) {
        paired = true;
        const int odd = lane & 1;
#pragma unroll
        for (int m = 0; m < VPL / 2; ++m) {
          keepk[2 * m] = keepk[2 * m + 1] = 0u;
          if (none_visible[j][2 * m] && none_visible[j][2 * m + 1] && !empty) continue;
          const int cpair = (c0 - odd) + (2 * m + odd) * cstride;  // the pair's even chunk
          const uint64_t flat = (uint64_t)row[j] * (uint64_t)g.sk + (uint64_t)cpair * E;
          const uint32_t bits = dropout_keep_bits(flat >> 3, d.seed, d.offset, d.threshold);
          const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(
              0, (int)bits, kDppQuadSwap1, 0xF, 0xF, false);
          const uint32_t mine = (bits >> (4 * odd)) & 0xFu;     // slot 2m + odd
          const uint32_t theirs = (other >> (4 * odd)) & 0xFu;  // the other slot
          keepk[2 * m] = odd ? theirs : mine;
          keepk[2 * m + 1] = odd ? mine : theirs;
        }
      }
    }
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (c < nchunks) {
        float o[E];
        if (none_visible[j][k]) {
#pragma unroll
          for (int e = 0; e < E; ++e) o[e] = fill;
        } else {
#pragma unroll
          for (int e = 0; e < E; ++e) o[e] = v[j][k][e] * inv + fill;
          // (the float value as it is: with a zero fill the product could
          //  otherwise be fused into the conversion to float16 in one build
          //  of the kernel and not in another, which differs on ties)
          if constexpr (kBias) {
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] = pinned(o[e]);
          }
        }
        if constexpr (DROP) {
          // exact zeros need no draw (wave-uniform test)
          if (!none_visible[j][k] || empty) {
            if constexpr (kPairDraw) {
              const uint32_t keep =
                  paired ? keepk[k] : chunk_keep_bits<E>(row[j], g.sk, c, d);
#pragma unroll
              for (int e = 0; e < E; ++e)
                o[e] = (keep >> e) & 1u ? o[e] * d.scale : 0.f;
            } else {
              const KeepWords<E> keep = chunk_keep_words<E>(row[j], g.sk, c, d);
#pragma unroll
              for (int e = 0; e < E; ++e)
                o[e] = keep.kept(e) ? o[e] * d.scale : 0.f;
            }
          }
        }
        store_chunk<T, E>(yr + (int64_t)c * E, o);
      }
    }
  }
}

// Backward of softmax + dropout from the saved logits: the probabilities are
// recomputed as exp2(x * scale * log2 e - stats[row][0]) * stats[row][1], the
// keep bits are regenerated from (seed, offset), and
// dx = scale * y * (dp - sum_k dp_k y_k) with dp = keep * dy / (1 - p).
template <typename T, int VPL, int RPW, int MODE, int LPR = kWave>
__global__ __launch_bounds__(1024) void softmax_dropout_bwd_kernel(
    const T *__restrict__ dy, const T *__restrict__ x,
    const float *__restrict__ stats, const uint8_t *__restrict__ mask,
    T *__restrict__ dx, SoftmaxGeom g, float scale, DropArgs d) {
  d = resolve_drop(d);
  constexpr int E = io<T>::EPV;
  constexpr uint32_t kAll = (1u << E) - 1u;
  __shared__ float red[16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rslot = g.wpr == 1 ? wave : wave / g.wpr;  // (uniform: the division is skipped)
  const int first = rslot * g.wpr;
  const int nchunks = g.sk / E;
  const int cstride = LPR == kWave ? kWave * g.wpr : LPR;
  constexpr int SUB = kWave / LPR;
  const int sl = LPR == kWave ? lane : (lane & (LPR - 1));
  const int c0 = (wave - first) * kWave + sl;
  const int64_t rbase = (work_block(g) * g.rpb + rslot) * (RPW * SUB) +
                        (LPR == kWave ? 0 : lane / LPR);
  const float c2 = scale * kLog2e;

  float yv[RPW][VPL][E], gv[RPW][VPL][E];
  uint32_t mbits[RPW][VPL];  // bit e set: key masked out
  int64_t row[RPW];
  bool rvalid[RPW];
  float rmax[RPW], rinv[RPW];
  constexpr bool kBias = MODE == kModeBias;
  float bv[kBias ? RPW : 1][kBias ? VPL : 1][kBias ? E : 1];
  const bool bias_f32 = g.bias_esize == 4;

#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int64_t r = rbase + j * SUB;
    rvalid[j] = r < g.rows;
    int visible = 0;
    const uint8_t *mrow = nullptr;
    row[j] = 0;
    rmax[j] = 0.f;
    rinv[j] = 0.f;
    if (rvalid[j]) {
      row_setup<MODE>(g, r, mask, row[j], visible, mrow);
      rmax[j] = stats[2 * row[j]];
      rinv[j] = stats[2 * row[j] + 1];
    }
    // uniform row: every key counts (with an additive term there is no such
    // convention: the probabilities are what the arithmetic gives)
    const bool empty = rinv[j] < 0.f && !kBias;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      uint32_t mb = kAll;
      if (rvalid[j] && c < nchunks) {
        if (empty) {
          mb = 0u;
        } else if constexpr (MODE == kModeCausal || MODE == kModeBias) {
          const int left = visible - c * E;
          mb = left >= E ? 0u : (left <= 0 ? mb : (mb & ~((1u << left) - 1u)));
        } else {
          mb = masked_chunk_bits<E>(mrow, c, visible);
        }
      }
      if constexpr (kBias) {
        if (mb != kAll) {
          load_bias_chunk<T, E>(mrow, c, bias_f32, bv[j][k]);
          // A chunk whose terms all absorb their logits has probability 0
          // throughout, unless the row's maximum is such a term itself (a
          // row without any other key): skip it altogether
          if (g.bias_skip && rmax[j] > kBiasHidden && bias_all_hidden<E>(bv[j][k]))
            mb = kAll;
        }
      }
      mbits[j][k] = mb;
    }
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const T *xr = x + row[j] * g.sk;
    const T *gr = dy + row[j] * g.sk;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (mbits[j][k] != kAll) {
        load_chunk<T, E>(xr + (int64_t)c * E, yv[j][k]);
        load_chunk<T, E>(gr + (int64_t)c * E, gv[j][k]);
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          yv[j][k][e] = 0.f;
          gv[j][k][e] = 0.f;
        }
      }
    }
  }
  bool none_loaded[RPW][VPL];
#pragma unroll
  for (int j = 0; j < RPW; ++j)
#pragma unroll
    for (int k = 0; k < VPL; ++k)
      none_loaded[j][k] = __builtin_amdgcn_ballot_w64(mbits[j][k] != kAll) == 0;

  float s[RPW];
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    float a = 0.f;
    const bool empty = rinv[j] < 0.f && !kBias;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      if (none_loaded[j][k]) continue;
      const int c = c0 + k * cstride;
      // (a chunk without a visible key was not loaded: its gradients are zeros
      //  whatever the draw says)
      const KeepWords<E> keep = chunk_keep_words<E>(row[j], g.sk, c, d);
      const float *bf = nullptr;
      if constexpr (kBias) bf = bv[j][k];
      // (the selects below stay per element: a wave-uniform branch around
      //  them for slots in which every lane sees all its keys measured 12 %
      //  slower at [256, 2048, 2048], 690 -> 772 us)
#pragma unroll
      for (int e = 0; e < E; ++e) {
        // the product is rounded before the subtraction, exactly as the
        // forward pass formed its exponent (no fused multiply-add here)
        float p;
        if constexpr (kBias) {
          // (the forward pass takes a term that absorbs its logit for the sum
          //  without reading the logit; the fused multiply-add returns that
          //  same term)
          const float u = __builtin_fmaf(yv[j][k][e], scale, bf[e]);
          p = __builtin_amdgcn_exp2f(mul_rn(sub_rn(u, rmax[j]), kLog2e)) * rinv[j];
        } else {
          p = __builtin_amdgcn_exp2f(sub_rn(mul_rn(yv[j][k][e], c2), rmax[j])) * rinv[j];
        }
        if (empty) p = -rinv[j];
        if ((mbits[j][k] >> e) & 1u) p = 0.f;
        const float dp = keep.kept(e) ? mul_rn(gv[j][k][e], d.scale) : 0.f;
        yv[j][k][e] = p;
        gv[j][k][e] = dp;
        a += p * dp;
      }
    }
    s[j] = a;
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j)
    s[j] = row_reduce_sum<LPR>(s[j], red, wave, first, g.wpr, lane);

#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    if (!rvalid[j]) continue;
    T *dxr = dx + row[j] * g.sk;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (c < nchunks) {
        float o[E];
        if (none_loaded[j][k]) {
#pragma unroll
          for (int e = 0; e < E; ++e) o[e] = 0.f;
        } else {
#pragma unroll
          for (int e = 0; e < E; ++e)
            o[e] = scale * (yv[j][k][e] * (gv[j][k][e] - s[j]));
        }
        store_chunk<T, E>(dxr + (int64_t)c * E, o);
      }
    }
  }
}

template <typename T, int VPL, int RPW, int MODE, int LPR = kWave>
__global__ __launch_bounds__(1024) void softmax_bwd_kernel(
    const T *__restrict__ dy, const T *__restrict__ y,
    const uint8_t *__restrict__ mask, T *__restrict__ dx, SoftmaxGeom g,
    float scale) {
  constexpr int E = io<T>::EPV;
  constexpr uint32_t kAll = (1u << E) - 1u;
  __shared__ float red[2][16];
  const int lane = threadIdx.x & 63;
  // the wave index is uniform: keep it (and the row arithmetic) in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rslot = g.wpr == 1 ? wave : wave / g.wpr;  // (uniform: the division is skipped)
  const int first = rslot * g.wpr;
  const int nchunks = g.sk / E;
  const int cstride = LPR == kWave ? kWave * g.wpr : LPR;
  constexpr int SUB = kWave / LPR;
  const int sl = LPR == kWave ? lane : (lane & (LPR - 1));
  const int c0 = (wave - first) * kWave + sl;

  const int64_t rbase = (work_block(g) * g.rpb + rslot) * (RPW * SUB) +
                        (LPR == kWave ? 0 : lane / LPR);

  float yv[RPW][VPL][E], gv[RPW][VPL][E];
  bool skip[RPW][VPL];
  int64_t row[RPW];
  bool rvalid[RPW];

#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int64_t r = rbase + j * SUB;
    rvalid[j] = r < g.rows;
    int visible = 0;
    const uint8_t *mrow = nullptr;
    row[j] = 0;
    if (rvalid[j]) row_setup<MODE>(g, r, mask, row[j], visible, mrow);
    float anyvis = 0.f;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      bool sk_ = true;
      if (rvalid[j] && c < nchunks) {
        if constexpr (MODE == kModeCausal) {
          sk_ = visible - c * E <= 0;
        } else if constexpr (MODE == kModeMasked) {
          sk_ = masked_chunk_bits<E>(mrow, c, visible) == kAll;
        } else if constexpr (MODE == kModeBias) {
          // beyond the diagonal, or every additive term of the chunk absorbs
          // its logit: the probabilities are zeros (unless the whole row is
          // like that, which the test below catches)
          sk_ = visible - c * E <= 0;
          if (!sk_) {
            float bf[E];
            load_bias_chunk<T, E>(mrow, c, g.bias_esize == 4, bf);
            sk_ = bias_all_hidden<E>(bf);
          }
        } else {
          sk_ = false;
        }
      }
      skip[j][k] = sk_;
      if (!sk_) anyvis = 1.f;
    }
    if constexpr (MODE != kModeDense) {
      // a row with no visible key holds the uniform distribution: read it all
      anyvis = row_reduce_max<LPR>(anyvis, red[0], wave, first, g.wpr, lane);
      if (g.wpr > 1) __syncthreads();
      if (anyvis == 0.f) {
#pragma unroll
        for (int k = 0; k < VPL; ++k)
          skip[j][k] = !(rvalid[j] && c0 + k * cstride < nchunks);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const T *yr = y + row[j] * g.sk;
    const T *gr = dy + row[j] * g.sk;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (!skip[j][k]) {
        load_chunk<T, E>(yr + (int64_t)c * E, yv[j][k]);
        load_chunk<T, E>(gr + (int64_t)c * E, gv[j][k]);
      } else {
#pragma unroll
        for (int e = 0; e < E; ++e) {
          yv[j][k][e] = 0.f;
          gv[j][k][e] = 0.f;
        }
      }
    }
  }
  // wave-uniform: no lane of the wave loaded chunk slot (j, k) -> no arithmetic
  bool none_loaded[RPW][VPL];
#pragma unroll
  for (int j = 0; j < RPW; ++j)
#pragma unroll
    for (int k = 0; k < VPL; ++k)
      none_loaded[j][k] = __builtin_amdgcn_ballot_w64(!skip[j][k]) == 0;

  float s[RPW];
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    float a = 0.f;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      if (none_loaded[j][k]) continue;
#pragma unroll
      for (int e = 0; e < E; ++e) a += yv[j][k][e] * gv[j][k][e];
    }
    s[j] = a;
  }
#pragma unroll
  for (int j = 0; j < RPW; ++j)
    s[j] = row_reduce_sum<LPR>(s[j], red[1], wave, first, g.wpr, lane);

#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    if (!rvalid[j]) continue;
    T *dxr = dx + row[j] * g.sk;
#pragma unroll
    for (int k = 0; k < VPL; ++k) {
      const int c = c0 + k * cstride;
      if (c < nchunks) {
        float o[E];
        if (none_loaded[j][k]) {
#pragma unroll
          for (int e = 0; e < E; ++e) o[e] = 0.f;
        } else {
#pragma unroll
          for (int e = 0; e < E; ++e)
            o[e] = scale * (yv[j][k][e] * (gv[j][k][e] - s[j]));
        }
        store_chunk<T, E>(dxr + (int64_t)c * E, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// generic kernels: any sk / alignment; one 256-thread workgroup per row,
// three passes over the (L2-resident) row.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float block_reduce_256(float v, float *sh, bool is_max) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = is_max ? wave_max(v) : wave_sum(v);
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  return is_max ? fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]))
                : (sh[0] + sh[1]) + (sh[2] + sh[3]);
}

template <typename T, int MODE, bool DROP>
__global__ __launch_bounds__(256) void softmax_fwd_generic_kernel(
    const T *__restrict__ x, const uint8_t *__restrict__ mask,
    T *__restrict__ y, float *__restrict__ stats, SoftmaxGeom g, float scale,
    DropArgs d) {
  d = resolve_drop(d);
  __shared__ float sh[4];
  const float ninf = -__builtin_inff();
  // log2-domain logits t = x * (scale * log2 e), the same rounded products
  // and differences as in the register kernel
  const float c2 = scale * kLog2e;
  for (int64_t r = blockIdx.x; r < g.rows; r += gridDim.x) {
    int64_t row;
    int visible;
    const uint8_t *mrow;
    row_setup<MODE>(g, r, mask, row, visible, mrow);
    const T *xr = x + row * g.sk;
    T *yr = y + row * g.sk;
    constexpr bool kBias = MODE == kModeBias;
    const bool bias_f32 = g.bias_esize == 4;
    auto is_hidden = [&](int i) {
      if constexpr (MODE == kModeMasked) return mrow[i] != 0 || i >= visible;
      return i >= visible;
    };
    // the logit of key i, and its exponent relative to the row maximum m
    auto logit = [&](int i) {
      if constexpr (kBias)
        return __builtin_fmaf(io<T>::from_scalar(xr[i]), scale, bias_at<T>(mrow, i, bias_f32));
      return mul_rn(io<T>::from_scalar(xr[i]), c2);
    };
    auto expo = [&](int i, float m) {
      const float d = sub_rn(logit(i), m);
      return kBias ? mul_rn(d, kLog2e) : d;
    };
    float m = ninf;
    for (int i = threadIdx.x; i < g.sk; i += 256)
      if (!is_hidden(i)) m = fmaxf(m, logit(i));
    m = block_reduce_256(m, sh, true);
    const bool empty = m == ninf && !kBias;
    float s = 0.f;
    for (int i = threadIdx.x; i < g.sk; i += 256)
      if (!is_hidden(i)) s += __builtin_amdgcn_exp2f(expo(i, m));
    s = block_reduce_256(s, sh, false);
    const float inv = empty ? 0.f : row_recip(s);
    const float fill = empty ? g.inv_sk : 0.f;
    for (int i = threadIdx.x; i < g.sk; i += 256) {
      float p = 0.f;
      if (!is_hidden(i)) p = __builtin_amdgcn_exp2f(expo(i, m));
      float o = p * inv + fill;
      // (a key beyond the diagonal is an exact zero in a NaN row, too)
      if (kBias && is_hidden(i)) o = 0.f;
      if constexpr (kBias) o = pinned(o);
      if constexpr (DROP)
        o = keep_element(row * g.sk + i, d) ? o * d.scale : 0.f;
      yr[i] = io<T>::to_scalar(o);
    }
    if constexpr (DROP) {
      if (threadIdx.x == 0) {
        // (a query that the diagonal leaves without any key: zeros above, and
        //  finite statistics for the backward pass)
        const bool nokey = kBias && visible <= 0;
        stats[2 * row] = empty || nokey ? 0.f : m;
        stats[2 * row + 1] = empty ? -fill : (nokey ? 0.f : inv);
      }
    }
  }
}

template <typename T, int MODE>
__global__ __launch_bounds__(256) void softmax_dropout_bwd_generic_kernel(
    const T *__restrict__ dy, const T *__restrict__ x,
    const float *__restrict__ stats, const uint8_t *__restrict__ mask,
    T *__restrict__ dx, SoftmaxGeom g, float scale, DropArgs d) {
  d = resolve_drop(d);
  __shared__ float sh[4];
  const float c2 = scale * kLog2e;
  for (int64_t r = blockIdx.x; r < g.rows; r += gridDim.x) {
    int64_t row;
    int visible;
    const uint8_t *mrow;
    row_setup<MODE>(g, r, mask, row, visible, mrow);
    const T *xr = x + row * g.sk;
    const T *gr = dy + row * g.sk;
    T *dxr = dx + row * g.sk;
    const float m = stats[2 * row], inv = stats[2 * row + 1];
    constexpr bool kBias = MODE == kModeBias;
    const bool bias_f32 = g.bias_esize == 4;
    const bool empty = inv < 0.f && !kBias;
    auto prob = [&](int i) {
      if (empty) return -inv;
      bool hidden = i >= visible;
      if constexpr (MODE == kModeMasked) hidden = hidden || mrow[i] != 0;
      if (hidden) return 0.f;
      if constexpr (kBias) {
        const float u =
            __builtin_fmaf(io<T>::from_scalar(xr[i]), scale, bias_at<T>(mrow, i, bias_f32));
        return __builtin_amdgcn_exp2f(mul_rn(sub_rn(u, m), kLog2e)) * inv;
      }
      return __builtin_amdgcn_exp2f(
                 sub_rn(mul_rn(io<T>::from_scalar(xr[i]), c2), m)) *
             inv;
    };
    auto dprob = [&](int i) {
      return keep_element(row * g.sk + i, d)
                 ? mul_rn(io<T>::from_scalar(gr[i]), d.scale)
                 : 0.f;
    };
    float s = 0.f;
    for (int i = threadIdx.x; i < g.sk; i += 256) s += prob(i) * dprob(i);
    s = block_reduce_256(s, sh, false);
    for (int i = threadIdx.x; i < g.sk; i += 256)
      dxr[i] = io<T>::to_scalar(scale * (prob(i) * (dprob(i) - s)));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_bwd_generic_kernel(
    const T *__restrict__ dy, const T *__restrict__ y, T *__restrict__ dx,
    int64_t rows, int sk, float scale) {
  __shared__ float sh[4];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const T *yr = y + r * sk;
    const T *gr = dy + r * sk;
    T *dxr = dx + r * sk;
    float s = 0.f;
    for (int i = threadIdx.x; i < sk; i += 256)
      s += io<T>::from_scalar(yr[i]) * io<T>::from_scalar(gr[i]);
    s = block_reduce_256(s, sh, false);
    for (int i = threadIdx.x; i < sk; i += 256) {
      const float yy = io<T>::from_scalar(yr[i]);
      dxr[i] = io<T>::to_scalar(scale * (yy * (io<T>::from_scalar(gr[i]) - s)));
    }
  }
}

// ---------------------------------------------------------------------------
// generic rows of at most kWaveRowMax keys: one wavefront per row, the row in
// registers, no LDS and no barrier.  A lane accesses EW consecutive keys at a
// time (lane l holds keys EW * (l + 64 k) ...): EW = 4 or 2 when the row
// length and the pointers allow 8- or 4-byte accesses, else 1 (any length and
// alignment).  The arithmetic is that of the kernels above, term for term.
// ---------------------------------------------------------------------------
constexpr int kWaveRowMax = 2048;  // 32 elements per lane and operand; builds for 256, 1024, 2048

template <typename T, int EW>
__device__ __forceinline__ void ld_small(const T *p, float *f) {
  if constexpr (EW == 1) {
    f[0] = io<T>::from_scalar(p[0]);
  } else {
    T t[EW];
    if constexpr (EW * sizeof(T) == 4) {
      const uint32_t raw = *reinterpret_cast<const uint32_t *>(p);
      __builtin_memcpy(t, &raw, 4);
    } else {
      static_assert(EW * sizeof(T) == 8, "at most 8 bytes per access");
      const u32x2 raw = *reinterpret_cast<const u32x2 *>(p);
      __builtin_memcpy(t, &raw, 8);
    }
#pragma unroll
    for (int e = 0; e < EW; ++e) f[e] = io<T>::from_scalar(t[e]);
  }
}

template <typename T, int EW>
__device__ __forceinline__ void st_small(T *p, const float *f) {
  if constexpr (EW == 1) {
    p[0] = io<T>::to_scalar(f[0]);
  } else {
    T t[EW];
#pragma unroll
    for (int e = 0; e < EW; ++e) t[e] = io<T>::to_scalar(f[e]);
    if constexpr (EW * sizeof(T) == 4) {
      uint32_t raw;
      __builtin_memcpy(&raw, t, 4);
      *reinterpret_cast<uint32_t *>(p) = raw;
    } else {
      u32x2 raw;
      __builtin_memcpy(&raw, t, 8);
      *reinterpret_cast<u32x2 *>(p) = raw;
    }
  }
}

// bit e set: key i0 + e is masked out (EW consecutive mask bytes, EW-aligned)
template <int EW>
__device__ __forceinline__ uint32_t ld_mask_small(const uint8_t *p) {
  if constexpr (EW == 1) {
    return p[0] != 0 ? 1u : 0u;
  } else if constexpr (EW == 2) {
    const uint32_t m = *reinterpret_cast<const uint16_t *>(p);
    return ((m & 0xffu) ? 1u : 0u) | ((m >> 8) ? 2u : 0u);
  } else {
    const uint32_t m = *reinterpret_cast<const uint32_t *>(p);
    uint32_t bits = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) bits |= ((m >> (8 * e)) & 0xffu) ? (1u << e) : 0u;
    return bits;
  }
}

// keep bits of the EW consecutive elements that start at flat index `flat`
// (a multiple of EW, so they lie inside one dropout group)
template <int EW>
__device__ __forceinline__ uint32_t keep_small(int64_t flat, const DropArgs &d) {
  return dropout_keep_bits((uint64_t)flat >> 3, d.seed, d.offset, d.threshold) >>
         (uint32_t)(flat & 7);
}

template <typename T, int MODE, bool DROP, int EW, int ROWMAX>
__global__ __launch_bounds__(256) void softmax_fwd_wave_kernel(
    const T *__restrict__ x, const uint8_t *__restrict__ mask,
    T *__restrict__ y, float *__restrict__ stats, SoftmaxGeom g, float scale,
    DropArgs d) {
  d = resolve_drop(d);
  constexpr int K = ROWMAX / kWave / EW;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float ninf = -__builtin_inff();
  const float c2 = scale * kLog2e;
  for (int64_t r = (int64_t)blockIdx.x * 4 + wave; r < g.rows;
       r += (int64_t)gridDim.x * 4) {
    int64_t row;
    int visible;
    const uint8_t *mrow;
    row_setup<MODE>(g, r, mask, row, visible, mrow);
    const T *xr = x + row * g.sk;
    T *yr = y + row * g.sk;
    constexpr bool kBias = MODE == kModeBias;
    const bool bias_f32 = g.bias_esize == 4;
    float v[K][EW];
    float m = ninf;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i0 = (lane + kWave * k) * EW;
#pragma unroll
      for (int e = 0; e < EW; ++e) v[k][e] = ninf;
      if (i0 < g.sk) {
        // keys beyond the diagonal are not loaded; with a mask tensor the
        // logits are requested together with the mask bytes (waiting for the
        // mask first measures 30 % slower than the loads it can save)
        uint32_t hid = 0;
        if constexpr (MODE == kModeMasked) hid = ld_mask_small<EW>(mrow + i0);
        const bool none = i0 >= visible;  // (visible == sk without a diagonal)
        if (!none) {
          float t[EW];
          ld_small<T, EW>(xr + i0, t);
#pragma unroll
          for (int e = 0; e < EW; ++e) {
            const bool hidden =
                MODE == kModeMasked ? (((hid >> e) & 1u) != 0 || i0 + e >= visible)
                                    : i0 + e >= visible;
            if (!hidden) {
              if constexpr (kBias)
                v[k][e] = __builtin_fmaf(t[e], scale, bias_at<T>(mrow, i0 + e, bias_f32));
              else
                v[k][e] = mul_rn(t[e], c2);
            }
            m = fmaxf(m, v[k][e]);
          }
        }
      }
    }
    m = wave_max(m);
    const bool empty = m == ninf && !kBias;
    const float off = empty ? 0.f : m;
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < EW; ++e) {
        float dd = sub_rn(v[k][e], off);
        if constexpr (kBias) dd = mul_rn(dd, kLog2e);
        const float p = __builtin_amdgcn_exp2f(dd);  // 0 for hidden keys
        v[k][e] = p;
        s += p;
      }
    s = wave_sum(s);
    const float inv = empty ? 0.f : row_recip(s);
    const float fill = empty ? g.inv_sk : 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i0 = (lane + kWave * k) * EW;
      if (i0 < g.sk) {
        float o[EW];
        uint32_t keep = 0xffu;
        if constexpr (DROP) keep = keep_small<EW>(row * g.sk + i0, d);
#pragma unroll
        for (int e = 0; e < EW; ++e) {
          o[e] = v[k][e] * inv + fill;
          // (a key beyond the diagonal is an exact zero in a NaN row, too)
          if (kBias && i0 + e >= visible) o[e] = 0.f;
          if constexpr (kBias) o[e] = pinned(o[e]);
          if constexpr (DROP) o[e] = (keep >> e) & 1u ? o[e] * d.scale : 0.f;
        }
        st_small<T, EW>(yr + i0, o);
      }
    }
    if constexpr (DROP) {
      if (lane == 0) {
        // (a query that the diagonal leaves without any key: zeros above, and
        //  finite statistics for the backward pass)
        const bool nokey = kBias && visible <= 0;
        stats[2 * row] = empty || nokey ? 0.f : m;
        stats[2 * row + 1] = empty ? -fill : (nokey ? 0.f : inv);
      }
    }
  }
}

template <typename T, int MODE, int EW, int ROWMAX>
__global__ __launch_bounds__(256) void softmax_dropout_bwd_wave_kernel(
    const T *__restrict__ dy, const T *__restrict__ x,
    const float *__restrict__ stats, const uint8_t *__restrict__ mask,
    T *__restrict__ dx, SoftmaxGeom g, float scale, DropArgs d) {
  d = resolve_drop(d);
  constexpr int K = ROWMAX / kWave / EW;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float c2 = scale * kLog2e;
  for (int64_t r = (int64_t)blockIdx.x * 4 + wave; r < g.rows;
       r += (int64_t)gridDim.x * 4) {
    int64_t row;
    int visible;
    const uint8_t *mrow;
    row_setup<MODE>(g, r, mask, row, visible, mrow);
    const T *xr = x + row * g.sk;
    const T *gr = dy + row * g.sk;
    T *dxr = dx + row * g.sk;
    const float m = stats[2 * row], inv = stats[2 * row + 1];
    constexpr bool kBias = MODE == kModeBias;
    const bool bias_f32 = g.bias_esize == 4;
    const bool empty = inv < 0.f && !kBias;
    float pv[K][EW], gv[K][EW];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i0 = (lane + kWave * k) * EW;
#pragma unroll
      for (int e = 0; e < EW; ++e) {
        pv[k][e] = 0.f;
        gv[k][e] = 0.f;
      }
      uint32_t hid = 0;
      bool none = true;
      if (i0 < g.sk) {
        if constexpr (MODE == kModeMasked) hid = ld_mask_small<EW>(mrow + i0);
        // keys beyond the diagonal contribute nothing and are not loaded
        // (a row without a visible key is uniform: every key counts)
        none = !empty && i0 >= visible;
      }
      if (!none) {
        float xt[EW], gt[EW];
        ld_small<T, EW>(xr + i0, xt);
        ld_small<T, EW>(gr + i0, gt);
        const uint32_t keep = keep_small<EW>(row * g.sk + i0, d);
#pragma unroll
        for (int e = 0; e < EW; ++e) {
          const bool hidden =
              MODE == kModeMasked ? (((hid >> e) & 1u) != 0 || i0 + e >= visible)
                                  : i0 + e >= visible;
          float p = 0.f;
          if (empty) {
            p = -inv;
          } else if (!hidden) {
            if constexpr (kBias) {
              const float u =
                  __builtin_fmaf(xt[e], scale, bias_at<T>(mrow, i0 + e, bias_f32));
              p = __builtin_amdgcn_exp2f(mul_rn(sub_rn(u, m), kLog2e)) * inv;
            } else {
              p = __builtin_amdgcn_exp2f(sub_rn(mul_rn(xt[e], c2), m)) * inv;
            }
          }
          pv[k][e] = p;
          // (a rounded product: fused into the subtraction below it would
          //  leave the product's rounding error where an exact zero belongs)
          gv[k][e] = (keep >> e) & 1u ? mul_rn(gt[e], d.scale) : 0.f;
          s += pv[k][e] * gv[k][e];
        }
      }
    }
    s = wave_sum(s);
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i0 = (lane + kWave * k) * EW;
      if (i0 < g.sk) {
        float o[EW];
#pragma unroll
        for (int e = 0; e < EW; ++e) o[e] = scale * (pv[k][e] * (gv[k][e] - s));
        st_small<T, EW>(dxr + i0, o);
      }
    }
  }
}

template <typename T, int EW, int ROWMAX>
__global__ __launch_bounds__(256) void softmax_bwd_wave_kernel(
    const T *__restrict__ dy, const T *__restrict__ y, T *__restrict__ dx,
    int64_t rows, int sk, float scale) {
  constexpr int K = ROWMAX / kWave / EW;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t r = (int64_t)blockIdx.x * 4 + wave; r < rows;
       r += (int64_t)gridDim.x * 4) {
    const T *yr = y + r * sk;
    const T *gr = dy + r * sk;
    T *dxr = dx + r * sk;
    float yv[K][EW], gv[K][EW];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i0 = (lane + kWave * k) * EW;
#pragma unroll
      for (int e = 0; e < EW; ++e) {
        yv[k][e] = 0.f;
        gv[k][e] = 0.f;
      }
      if (i0 < sk) {
        ld_small<T, EW>(yr + i0, yv[k]);
        ld_small<T, EW>(gr + i0, gv[k]);
      }
#pragma unroll
      for (int e = 0; e < EW; ++e) s += yv[k][e] * gv[k][e];
    }
    s = wave_sum(s);
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int i0 = (lane + kWave * k) * EW;
      if (i0 < sk) {
        float o[EW];
#pragma unroll
        for (int e = 0; e < EW; ++e) o[e] = scale * (yv[k][e] * (gv[k][e] - s));
        st_small<T, EW>(dxr + i0, o);
      }
    }
  }
}

// Elements per access of the wave-per-row kernels: the widest of 4, 2, 1 for
// which the row length divides, an access stays within 8 bytes and every
// pointer (and the mask) is aligned to the access.
template <typename T>
static inline int wave_row_ew(int64_t sk, const void *a, const void *b,
                              const void *c, const uint8_t *mask) {
  for (int ew = 4; ew > 1; ew >>= 1) {
    const uintptr_t bytes = (uintptr_t)ew * sizeof(T);
    if (bytes > 8 || sk % ew != 0) continue;
    const uintptr_t all = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                          reinterpret_cast<uintptr_t>(c);
    if ((all & (bytes - 1)) != 0) continue;
    if (mask != nullptr && (reinterpret_cast<uintptr_t>(mask) & (uintptr_t)(ew - 1)) != 0) continue;
    return ew;
  }
  return 1;
}

// workgroups of a wave-per-row launch (four rows each)
static inline int64_t wave_row_grid(int64_t rows) {
  const int64_t want = ceil_div(rows, 4);
  const int64_t cap = (int64_t)device_cu_count() * 64;
  return want < cap ? want : cap;
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct SoftmaxPlan {
  int vpl, rpw, wpr, rpb;
  int lpr;  // lanes that hold a row: 64, or 8 / 16 / 32 for short rows
  bool ok;
};

// max_elems: elements of one operand a lane may hold (register budget).
static SoftmaxPlan plan_softmax(int64_t sk, int E, int max_elems,
                                int default_rpw, int one_chunk_rpw,
                                bool two_chunk_groups = false) {
  SoftmaxPlan p{0, 1, 1, 1, kWave, false};
  if (sk % E != 0) return p;
  const int64_t nchunks = sk / E;
  const int maxvpl = max_elems / E;  // 8 or 4 for 16-bit types, 16 or 8 for fp32
  int64_t wpr = ceil_div(nchunks, (int64_t)kWave * (maxvpl > 8 ? 8 : maxvpl));
  if (wpr > 16) return p;
  const int64_t need = ceil_div(nchunks, kWave * wpr);
  int vpl = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 8;
  int rpw = 1;
  // short rows: several rows side by side in a wave instead of idle lanes
  if (nchunks <= 32 && g_tune.softmax_lanes_per_row != kWave) {
    p.lpr = nchunks <= 8 ? 8 : nchunks <= 16 ? 16 : 32;
    if (g_tune.softmax_lanes_per_row == 8 || g_tune.softmax_lanes_per_row == 16 ||
        g_tune.softmax_lanes_per_row == 32)
      if (g_tune.softmax_lanes_per_row >= p.lpr) p.lpr = g_tune.softmax_lanes_per_row;
  }
  // rows of exactly 3 x 8 / 16 / 32 / 64 chunks (192, 384, 768, 1536 16-bit
  // keys): three chunks per lane, no idle lane
  if (nchunks % 3 == 0 && g_tune.softmax_lanes_per_row != kWave && 3 * E <= max_elems) {
    const int64_t q = nchunks / 3;
    if (q == 8 || q == 16 || q == 32 || q == 64) {
      p.vpl = 3;
      p.rpw = 1;
      p.wpr = 1;
      p.rpb = g_tune.softmax_rows_per_block > 0 ? g_tune.softmax_rows_per_block : 4;
      p.lpr = (int)q;
      p.ok = true;
      return p;
    }
  }
  // forward: rows of exactly 2 x 8 / 16 / 32 chunks (128, 256, 512 16-bit
  // keys) as two chunks per lane in a lane group
  if (two_chunk_groups && nchunks % 2 == 0 && g_tune.softmax_lanes_per_row != kWave &&
      g_tune.softmax_lanes_per_row != 1) {
    const int64_t q = nchunks / 2;
    if (q == 8 || q == 16 || q == 32) {
      // one row set per wave without a mask tensor, two with one (measured)
      int want = g_tune.softmax_rows_per_wave > 0 ? g_tune.softmax_rows_per_wave : default_rpw;
      p.vpl = 2;
      p.rpw = want >= 2 && 2 * 2 * E <= max_elems ? 2 : 1;
      p.wpr = 1;
      // (one wave per workgroup: 6 % faster at sequence length 128)
      p.rpb = g_tune.softmax_rows_per_block > 0 ? g_tune.softmax_rows_per_block : 1;
      p.lpr = (int)q;
      p.ok = true;
      return p;
    }
  }
  if (wpr == 1) {
    // row sets a wave handles at once; measured best on MI355X: one, or two
    // for the forward with a mask tensor (its loads wait for the mask bytes);
    // a forward that holds one chunk per lane (rows of up to 512 16-bit
    // keys) wants four, which hides its two dependent reductions
    int want = g_tune.softmax_rows_per_wave > 0
                   ? g_tune.softmax_rows_per_wave
                   : (vpl == 1 ? one_chunk_rpw : default_rpw);
    rpw = want >= 4 ? 4 : (want >= 2 ? 2 : 1);
    while (rpw > 1 && (rpw * vpl * E > max_elems || rpw * vpl > 8)) rpw >>= 1;
  }
  p.vpl = vpl;
  p.rpw = rpw;
  p.wpr = (int)wpr;
  // one row (set) per workgroup: workgroups of a single wave measure 3-6 %
  // faster on MI355X than four waves that each own a row (bf16 [256,2048,2048]
  // causal forward 570 -> 537 us, backward 744 -> 707 us)
  p.rpb = wpr == 1 || wpr >= 4 ? 1 : (int)(4 / wpr);
  if (g_tune.softmax_rows_per_block > 0) p.rpb = g_tune.softmax_rows_per_block;
  while (p.rpb * p.wpr > 16) --p.rpb;
  p.ok = true;
  return p;
}

constexpr int kFwdMaxElems = 64;  // one operand resident
constexpr int kBwdMaxElems = 32;  // two operands resident

#define OSLO_SM_CASES_LPR(LAUNCH, LPR_)    \
  if (pl.rpw == 1) {                       \
    LAUNCH(1, 1, LPR_);                    \
  } else if (pl.rpw == 2) {                \
    LAUNCH(1, 2, LPR_);                    \
  } else {                                 \
    LAUNCH(1, 4, LPR_);                    \
  }
#define OSLO_SM_CASES(LAUNCH)              \
  if (pl.vpl == 3 && pl.lpr == 8) {        \
    LAUNCH(3, 1, 8);                       \
  } else if (pl.vpl == 3 && pl.lpr == 16) { \
    LAUNCH(3, 1, 16);                      \
  } else if (pl.vpl == 3 && pl.lpr == 32) { \
    LAUNCH(3, 1, 32);                      \
  } else if (pl.vpl == 3) {                \
    LAUNCH(3, 1, kWave);                   \
  } else if (pl.vpl == 2 && pl.lpr == 8 && pl.rpw == 1) {  \
    LAUNCH(2, 1, 8);                       \
  } else if (pl.vpl == 2 && pl.lpr == 8) { \
    LAUNCH(2, 2, 8);                       \
  } else if (pl.vpl == 2 && pl.lpr == 16 && pl.rpw == 1) { \
    LAUNCH(2, 1, 16);                      \
  } else if (pl.vpl == 2 && pl.lpr == 16) { \
    LAUNCH(2, 2, 16);                      \
  } else if (pl.vpl == 2 && pl.lpr == 32 && pl.rpw == 1) { \
    LAUNCH(2, 1, 32);                      \
  } else if (pl.vpl == 2 && pl.lpr == 32) { \
    LAUNCH(2, 2, 32);                      \
  } else if (pl.lpr == 8) {                \
    OSLO_SM_CASES_LPR(LAUNCH, 8)           \
  } else if (pl.lpr == 16) {               \
    OSLO_SM_CASES_LPR(LAUNCH, 16)          \
  } else if (pl.lpr == 32) {               \
    OSLO_SM_CASES_LPR(LAUNCH, 32)          \
  } else if (pl.vpl == 1 && pl.rpw == 1) { \
    LAUNCH(1, 1, kWave);                   \
  } else if (pl.vpl == 1 && pl.rpw == 2) { \
    LAUNCH(1, 2, kWave);                   \
  } else if (pl.vpl == 1 && pl.rpw == 4) { \
    LAUNCH(1, 4, kWave);                   \
  } else if (pl.vpl == 2 && pl.rpw == 1) { \
    LAUNCH(2, 1, kWave);                   \
  } else if (pl.vpl == 2 && pl.rpw == 2) { \
    LAUNCH(2, 2, kWave);                   \
  } else if (pl.vpl == 2 && pl.rpw == 4) { \
    LAUNCH(2, 4, kWave);                   \
  } else if (pl.vpl == 4 && pl.rpw == 1) { \
    LAUNCH(4, 1, kWave);                   \
  } else if (pl.vpl == 4 && pl.rpw == 2) { \
    LAUNCH(4, 2, kWave);                   \
  } else {                                 \
    LAUNCH(8, 1, kWave);                   \
  }

// The (chunks per lane, row sets per wave, lanes per row) triples that the
// plan of a backward pass can come out with: at most 32 resident elements of
// each operand per lane in a 16-bit type and 16 in fp32 (32 only for rows that
// need eight chunks per lane, which take one row set), and two chunks per lane
// in a lane group only in the forward pass.  Other triples are not built.
template <typename T>
constexpr bool bwd_plan_reaches(int vpl, int rpw, int lpr) {
  constexpr int E = io<T>::EPV;
  if (vpl == 2 && lpr < kWave) return false;
  if (sizeof(T) == 4) return vpl * rpw * E <= 16 || (vpl == 8 && rpw == 1);
  return vpl * rpw * E <= kBwdMaxElems;
}

// The register kernels read the additive term in 16-byte vectors: its base
// address and the byte offsets of its rows must be multiples of 16.
static inline bool bias_vec_ok(const SoftmaxGeom &g, const uint8_t *bias) {
  if (bias == nullptr) return true;
  const int64_t es = g.bias_esize;
  return aligned16(bias) && (g.bias_sb * es) % 16 == 0 && (g.bias_sh * es) % 16 == 0 &&
         (g.bias_sq * es) % 16 == 0;
}

// elements of one operand per lane the kernels with an additive term hold at
// most (the term's chunks stay resident next to the logits)
constexpr int kBiasMaxElems = 32;

// stats != nullptr selects the dropout variant (d is ignored otherwise).
template <typename T, int MODE>
int launch_softmax_fwd(const void *x, const uint8_t *mask, void *y,
                              float *stats, DropArgs d, SoftmaxGeom g,
                              float scale, hipStream_t st) {
  constexpr int E = io<T>::EPV;
  set_fast_div(g);
  const bool drop = stats != nullptr;
  // 64 bytes of the operand per lane (32 16-bit or 16 fp32 elements) measure
  // 10-25 % faster than twice that (rows of 4096 and more 16-bit keys then
  // take two or more waves); 64 elements only where a row would otherwise not
  // fit one workgroup
  const int cap = g_tune.softmax_fwd_elems > 0 ? g_tune.softmax_fwd_elems
                                               : (sizeof(T) == 4 ? 16 : 32);
  // (two row sets per wave where the loads of the logits wait for mask bytes;
  //  with an additive term one measures faster, 186 against 232 us at
  //  [16,16,1024,1024] fp16, whether or not the loads wait for the term)
  const int default_rpw = MODE == kModeMasked ? 2 : 1;
  SoftmaxPlan pl = plan_softmax(g.sk, E, cap, default_rpw, 4, true);
  if (!pl.ok && cap < kFwdMaxElems && MODE != kModeBias)
    pl = plan_softmax(g.sk, E, kFwdMaxElems, default_rpw, 4);
  if (MODE == kModeBias && pl.ok && pl.vpl * pl.rpw * E > kBiasMaxElems) pl.ok = false;
  const bool vec_ok = pl.ok && aligned16(x) && aligned16(y) &&
                      (MODE != kModeMasked ||
                       (reinterpret_cast<uintptr_t>(mask) % E) == 0) &&
                      (MODE != kModeBias || bias_vec_ok(g, mask));
  if (!vec_ok) {
    const int64_t grid = g.rows < (int64_t)device_cu_count() * 32
                             ? g.rows
                             : (int64_t)device_cu_count() * 32;
    if (g.sk <= kWaveRowMax) {
      const dim3 wgrid((unsigned)wave_row_grid(g.rows));
      const int ew = wave_row_ew<T>(g.sk, x, y, nullptr, MODE == kModeMasked ? mask : nullptr);
#define OSLO_SM_WAVE_FWD_R(EW_, RM_)                                       \
  do {                                                                     \
    if constexpr (EW_ * sizeof(T) <= 8) {                                  \
      if (drop)                                                            \
        softmax_fwd_wave_kernel<T, MODE, true, EW_, RM_><<<wgrid, 256, 0, st>>>(  \
            (const T *)x, mask, (T *)y, stats, g, scale, d);               \
      else                                                                 \
        softmax_fwd_wave_kernel<T, MODE, false, EW_, RM_><<<wgrid, 256, 0, st>>>( \
            (const T *)x, mask, (T *)y, nullptr, g, scale, d);             \
    }                                                                      \
  } while (0)
#define OSLO_SM_WAVE_FWD(EW_)                                              \
  do {                                                                     \
    if (g.sk <= 256) OSLO_SM_WAVE_FWD_R(EW_, 256);                         \
    else if (g.sk <= 1024) OSLO_SM_WAVE_FWD_R(EW_, 1024);                  \
    else OSLO_SM_WAVE_FWD_R(EW_, 2048);                                    \
  } while (0)
      if (ew == 4) OSLO_SM_WAVE_FWD(4);
      else if (ew == 2) OSLO_SM_WAVE_FWD(2);
      else OSLO_SM_WAVE_FWD(1);
#undef OSLO_SM_WAVE_FWD
#undef OSLO_SM_WAVE_FWD_R
      return check_launch("softmax_fwd_wave_kernel");
    }
    if (drop)
      softmax_fwd_generic_kernel<T, MODE, true>
          <<<dim3((unsigned)grid), 256, 0, st>>>((const T *)x, mask, (T *)y,
                                                 stats, g, scale, d);
    else
      softmax_fwd_generic_kernel<T, MODE, false>
          <<<dim3((unsigned)grid), 256, 0, st>>>((const T *)x, mask, (T *)y,
                                                 nullptr, g, scale, d);
    return check_launch("softmax_fwd_generic_kernel");
  }
  g.wpr = pl.wpr;
  // (rows of several waves run faster in stored order: sequence 4096, 3-12 %)
  if (g_tune.softmax_causal_order == 0 && pl.wpr > 1) g.causal_order = 1;
  g.rpb = pl.rpb;
  const int threads = kWave * pl.wpr * pl.rpb;
  const int64_t nblocks =
      ceil_div(g.rows, (int64_t)pl.rpb * pl.rpw * (kWave / pl.lpr));
  const int64_t per_launch = max_workgroups(threads);
#define OSLO_SM_FWD(VPL, RPW, LPR_)                                  \
  if constexpr (VPL * RPW * E <= (MODE == kModeBias ? kBiasMaxElems : kFwdMaxElems)) { \
    if (drop)                                                        \
      softmax_fwd_kernel<T, VPL, RPW, MODE, true, LPR_>              \
          <<<dim3((unsigned)grid), threads, 0, st>>>(                \
              (const T *)x, mask, (T *)y, stats, g, scale, d);       \
    else                                                             \
      softmax_fwd_kernel<T, VPL, RPW, MODE, false, LPR_>             \
          <<<dim3((unsigned)grid), threads, 0, st>>>(                \
              (const T *)x, mask, (T *)y, nullptr, g, scale, d);     \
  } else                                                             \
    return fail(OSLO_ERR_UNSUPPORTED, "softmax fwd: no kernel for %d x %d chunks per lane", VPL, RPW)
  // (rows of a term shared by the batch: one die per run of consecutive blocks)
  int64_t launch_blocks = nblocks;
  if (MODE == kModeBias && g.batch_inner && g_tune.softmax_bias_order == 3 &&
      nblocks >= 64 && nblocks + 8 <= per_launch) {
    g.xcd_wpx = ceil_div(nblocks, 8);
    launch_blocks = 8 * g.xcd_wpx;
  }
  for (g.blk0 = 0; g.blk0 < launch_blocks; g.blk0 += per_launch) {
    const int64_t grid = launch_blocks - g.blk0 < per_launch ? launch_blocks - g.blk0 : per_launch;
    OSLO_SM_CASES(OSLO_SM_FWD)
    const int rc = check_launch("softmax_fwd_kernel");
    if (rc != OSLO_OK) return rc;
  }
#undef OSLO_SM_FWD
  return OSLO_OK;
}

template <typename T, int MODE>
int launch_softmax_bwd(const void *dy, const void *y,
                              const uint8_t *mask, void *dx, SoftmaxGeom g,
                              float scale, hipStream_t st) {
  constexpr int E = io<T>::EPV;
  set_fast_div(g);
  // (fp32: 16 elements of each operand per lane, as in the forward)
  SoftmaxPlan pl = plan_softmax(g.sk, E, sizeof(T) == 4 ? 16 : kBwdMaxElems, 1, 1);
  if (!pl.ok && sizeof(T) == 4) pl = plan_softmax(g.sk, E, kBwdMaxElems, 1, 1);
  const bool vec_ok = pl.ok && aligned16(dy) && aligned16(y) &&
                      aligned16(dx) &&
                      (MODE != kModeMasked ||
                       (reinterpret_cast<uintptr_t>(mask) % E) == 0) &&
                      (MODE != kModeBias || bias_vec_ok(g, mask));
  if (!vec_ok) {
    const int64_t grid = g.rows < (int64_t)device_cu_count() * 32
                             ? g.rows
                             : (int64_t)device_cu_count() * 32;
    if (g.sk <= kWaveRowMax) {
      const dim3 wgrid((unsigned)wave_row_grid(g.rows));
      const int ew = wave_row_ew<T>(g.sk, dy, y, dx, nullptr);
#define OSLO_SM_WAVE_BWD_R(EW_, RM_)                                       \
  do {                                                                     \
    if constexpr (EW_ * sizeof(T) <= 8)                                    \
      softmax_bwd_wave_kernel<T, EW_, RM_><<<wgrid, 256, 0, st>>>(         \
          (const T *)dy, (const T *)y, (T *)dx, g.rows, g.sk, scale);      \
  } while (0)
#define OSLO_SM_WAVE_BWD(EW_)                                              \
  do {                                                                     \
    if (g.sk <= 256) OSLO_SM_WAVE_BWD_R(EW_, 256);                         \
    else if (g.sk <= 1024) OSLO_SM_WAVE_BWD_R(EW_, 1024);                  \
    else OSLO_SM_WAVE_BWD_R(EW_, 2048);                                    \
  } while (0)
      if (ew == 4) OSLO_SM_WAVE_BWD(4);
      else if (ew == 2) OSLO_SM_WAVE_BWD(2);
      else OSLO_SM_WAVE_BWD(1);
#undef OSLO_SM_WAVE_BWD
#undef OSLO_SM_WAVE_BWD_R
      return check_launch("softmax_bwd_wave_kernel");
    }
    softmax_bwd_generic_kernel<T><<<dim3((unsigned)grid), 256, 0, st>>>(
        (const T *)dy, (const T *)y, (T *)dx, g.rows, g.sk, scale);
    return check_launch("softmax_bwd_generic_kernel");
  }
  g.wpr = pl.wpr;
  // (rows of several waves run faster in stored order: sequence 4096, 3-12 %)
  if (g_tune.softmax_causal_order == 0 && pl.wpr > 1) g.causal_order = 1;
  g.rpb = pl.rpb;
  const int threads = kWave * pl.wpr * pl.rpb;
  const int64_t nblocks =
      ceil_div(g.rows, (int64_t)pl.rpb * pl.rpw * (kWave / pl.lpr));
  const int64_t per_launch = max_workgroups(threads);
#define OSLO_SM_BWD(VPL, RPW, LPR_)                        \
  if constexpr (bwd_plan_reaches<T>(VPL, RPW, LPR_))       \
    softmax_bwd_kernel<T, VPL, RPW, MODE, LPR_>            \
        <<<dim3((unsigned)grid), threads, 0, st>>>(        \
            (const T *)dy, (const T *)y, mask, (T *)dx, g, scale); \
  else                                                     \
    return fail(OSLO_ERR_UNSUPPORTED, "softmax bwd: no kernel for %d x %d chunks per lane", VPL, RPW)
  for (g.blk0 = 0; g.blk0 < nblocks; g.blk0 += per_launch) {
    const int64_t grid = nblocks - g.blk0 < per_launch ? nblocks - g.blk0 : per_launch;
    OSLO_SM_CASES(OSLO_SM_BWD)
    const int rc = check_launch("softmax_bwd_kernel");
    if (rc != OSLO_OK) return rc;
  }
#undef OSLO_SM_BWD
  return OSLO_OK;
}

template <typename T, int MODE>
int launch_softmax_dropout_bwd(const void *dy, const void *x,
                                      const float *stats, const uint8_t *mask,
                                      void *dx, DropArgs d, SoftmaxGeom g,
                                      float scale, hipStream_t st) {
  constexpr int E = io<T>::EPV;
  set_fast_div(g);
  // (fp32: 16 elements of each operand per lane, as in the forward)
  SoftmaxPlan pl = plan_softmax(g.sk, E, sizeof(T) == 4 ? 16 : kBwdMaxElems, 1, 1);
  if (!pl.ok && sizeof(T) == 4) pl = plan_softmax(g.sk, E, kBwdMaxElems, 1, 1);
  // (with an additive term resident next to the two operands, four row sets
  //  per wave no longer fit the register budget)
  if (MODE == kModeBias && pl.rpw > 2) pl.rpw = 2;
  const bool vec_ok = pl.ok && aligned16(dy) && aligned16(x) && aligned16(dx) &&
                      (MODE != kModeMasked ||
                       (reinterpret_cast<uintptr_t>(mask) % E) == 0) &&
                      (MODE != kModeBias || bias_vec_ok(g, mask));
  if (!vec_ok) {
    const int64_t grid = g.rows < (int64_t)device_cu_count() * 32
                             ? g.rows
                             : (int64_t)device_cu_count() * 32;
    if (g.sk <= kWaveRowMax) {
      const dim3 wgrid((unsigned)wave_row_grid(g.rows));
      const int ew = wave_row_ew<T>(g.sk, dy, x, dx, MODE == kModeMasked ? mask : nullptr);
#define OSLO_SM_WAVE_DBWD_R(EW_, RM_)                                      \
  do {                                                                     \
    if constexpr (EW_ * sizeof(T) <= 8)                                    \
      softmax_dropout_bwd_wave_kernel<T, MODE, EW_, RM_><<<wgrid, 256, 0, st>>>( \
          (const T *)dy, (const T *)x, stats, mask, (T *)dx, g, scale, d); \
  } while (0)
#define OSLO_SM_WAVE_DBWD(EW_)                                             \
  do {                                                                     \
    if (g.sk <= 256) OSLO_SM_WAVE_DBWD_R(EW_, 256);                        \
    else if (g.sk <= 1024) OSLO_SM_WAVE_DBWD_R(EW_, 1024);                 \
    else OSLO_SM_WAVE_DBWD_R(EW_, 2048);                                   \
  } while (0)
      if (ew == 4) OSLO_SM_WAVE_DBWD(4);
      else if (ew == 2) OSLO_SM_WAVE_DBWD(2);
      else OSLO_SM_WAVE_DBWD(1);
#undef OSLO_SM_WAVE_DBWD
#undef OSLO_SM_WAVE_DBWD_R
      return check_launch("softmax_dropout_bwd_wave_kernel");
    }
    softmax_dropout_bwd_generic_kernel<T, MODE>
        <<<dim3((unsigned)grid), 256, 0, st>>>((const T *)dy, (const T *)x,
                                               stats, mask, (T *)dx, g, scale,
                                               d);
    return check_launch("softmax_dropout_bwd_generic_kernel");
  }
  g.wpr = pl.wpr;
  // (rows of several waves run faster in stored order: sequence 4096, 3-12 %)
  if (g_tune.softmax_causal_order == 0 && pl.wpr > 1) g.causal_order = 1;
  g.rpb = pl.rpb;
  const int threads = kWave * pl.wpr * pl.rpb;
  const int64_t nblocks =
      ceil_div(g.rows, (int64_t)pl.rpb * pl.rpw * (kWave / pl.lpr));
  const int64_t per_launch = max_workgroups(threads);
#define OSLO_SM_DBWD(VPL, RPW, LPR_)                                \
  if constexpr (bwd_plan_reaches<T>(VPL, RPW, LPR_) && (MODE != kModeBias || RPW <= 2)) \
    softmax_dropout_bwd_kernel<T, VPL, RPW, MODE, LPR_>             \
        <<<dim3((unsigned)grid), threads, 0, st>>>(                 \
            (const T *)dy, (const T *)x, stats, mask, (T *)dx, g,   \
            scale, d);                                              \
  else                                                              \
    return fail(OSLO_ERR_UNSUPPORTED, "softmax dropout bwd: no kernel for %d x %d chunks per lane", VPL, RPW)
  // (rows of a term shared by the batch: one die per run of consecutive blocks)
  int64_t launch_blocks = nblocks;
  if (MODE == kModeBias && g.batch_inner && g_tune.softmax_bias_order == 3 &&
      nblocks >= 64 && nblocks + 8 <= per_launch) {
    g.xcd_wpx = ceil_div(nblocks, 8);
    launch_blocks = 8 * g.xcd_wpx;
  }
  for (g.blk0 = 0; g.blk0 < launch_blocks; g.blk0 += per_launch) {
    const int64_t grid = launch_blocks - g.blk0 < per_launch ? launch_blocks - g.blk0 : per_launch;
    OSLO_SM_CASES(OSLO_SM_DBWD)
    const int rc = check_launch("softmax_dropout_bwd_kernel");
    if (rc != OSLO_OK) return rc;
  }
#undef OSLO_SM_DBWD
  return OSLO_OK;
}

// Every (type, mode) pair of the three launchers, as explicit instantiations:
// softmax_inst.hip defines them, one type and one direction per translation
// unit (so that the units build in parallel), softmax.hip declares them extern.
#define OSLO_SM_FWD_INSTANCES(PREFIX, T)                                                   \
  PREFIX template int launch_softmax_fwd<T, kModeCausal>(const void *, const uint8_t *, void *, \
      float *, DropArgs, SoftmaxGeom, float, hipStream_t);                                 \
  PREFIX template int launch_softmax_fwd<T, kModeMasked>(const void *, const uint8_t *, void *, \
      float *, DropArgs, SoftmaxGeom, float, hipStream_t);                                 \
  PREFIX template int launch_softmax_fwd<T, kModeBias>(const void *, const uint8_t *, void *, \
      float *, DropArgs, SoftmaxGeom, float, hipStream_t);
#define OSLO_SM_BWD_ONE(PREFIX, T, MODE)                                                   \
  PREFIX template int launch_softmax_bwd<T, MODE>(const void *, const void *, const uint8_t *, \
      void *, SoftmaxGeom, float, hipStream_t);
#define OSLO_SM_DBWD_ONE(PREFIX, T, MODE)                                                  \
  PREFIX template int launch_softmax_dropout_bwd<T, MODE>(const void *, const void *,      \
      const float *, const uint8_t *, void *, DropArgs, SoftmaxGeom, float, hipStream_t);
#define OSLO_SM_BWD_INSTANCES(PREFIX, T)   \
  OSLO_SM_BWD_ONE(PREFIX, T, kModeCausal)  \
  OSLO_SM_BWD_ONE(PREFIX, T, kModeMasked)  \
  OSLO_SM_BWD_ONE(PREFIX, T, kModeDense)   \
  OSLO_SM_BWD_ONE(PREFIX, T, kModeBias)    \
  OSLO_SM_DBWD_ONE(PREFIX, T, kModeCausal) \
  OSLO_SM_DBWD_ONE(PREFIX, T, kModeMasked) \
  OSLO_SM_DBWD_ONE(PREFIX, T, kModeBias)

}  // namespace oslo
