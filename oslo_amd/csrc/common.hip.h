// Device-side building blocks shared by every kernel of liboslo_hip.so:
// 128-bit global loads/stores, dtype packing, wave64 DPP reductions and the
// Philox4x32-10 generator.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace oslo {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// 128-bit global memory access.  Activations are streamed exactly once, so
// they bypass cache retention with the non-temporal hint; small reused
// vectors (gamma, beta, bias) use ordinary loads and stay in L2.
// ---------------------------------------------------------------------------
__device__ __forceinline__ u32x4 ld16_stream(const void *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
__device__ __forceinline__ void st16_stream(void *p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ u32x4 ld16_cached(const void *p) {
  return *reinterpret_cast<const u32x4 *>(p);
}

// ---------------------------------------------------------------------------
// dtype traits: EPV = elements per 16-byte vector.
// ---------------------------------------------------------------------------
template <typename T> struct io;

template <> struct io<float> {
  static constexpr int EPV = 4;
  static __device__ __forceinline__ void unpack(u32x4 r, float *f) {
    f[0] = __uint_as_float(r.x);
    f[1] = __uint_as_float(r.y);
    f[2] = __uint_as_float(r.z);
    f[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    u32x4 r;
    r.x = __float_as_uint(f[0]);
    r.y = __float_as_uint(f[1]);
    r.z = __float_as_uint(f[2]);
    r.w = __float_as_uint(f[3]);
    return r;
  }
  static __device__ __forceinline__ float round(float v) { return v; }
  static __device__ __forceinline__ float from_scalar(float v) { return v; }
  static __device__ __forceinline__ float to_scalar(float v) { return v; }
};

template <> struct io<__bf16> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ void unpack(u32x4 r, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(r[i] << 16);
      f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    f32x2 v;
    v.x = a;
    v.y = b;
    bf16x2 h = __builtin_convertvector(v, bf16x2);  // v_cvt_pk_bf16_f32, RNE
    return __builtin_bit_cast(uint32_t, h);
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = pack2(f[2 * i], f[2 * i + 1]);
    return r;
  }
  static __device__ __forceinline__ float round(float v) {
    return static_cast<float>(static_cast<__bf16>(v));
  }
  static __device__ __forceinline__ float from_scalar(__bf16 v) {
    return static_cast<float>(v);
  }
  static __device__ __forceinline__ __bf16 to_scalar(float v) {
    return static_cast<__bf16>(v);
  }
};

template <> struct io<_Float16> {
  static constexpr int EPV = 8;
  static __device__ __forceinline__ void unpack(u32x4 r, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // copy the element first: a bit_cast straight from the vector-element
      // lvalue r[i] reads element 0 with this compiler
      const uint32_t w = r[i];
      f16x2 h = __builtin_bit_cast(f16x2, w);
      f[2 * i] = static_cast<float>(h.x);
      f[2 * i + 1] = static_cast<float>(h.y);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f16x2 h;
      h.x = static_cast<_Float16>(f[2 * i]);  // v_cvt_f16_f32, RNE
      h.y = static_cast<_Float16>(f[2 * i + 1]);
      r[i] = __builtin_bit_cast(uint32_t, h);
    }
    return r;
  }
  static __device__ __forceinline__ float round(float v) {
    return static_cast<float>(static_cast<_Float16>(v));
  }
  static __device__ __forceinline__ float from_scalar(_Float16 v) {
    return static_cast<float>(v);
  }
  static __device__ __forceinline__ _Float16 to_scalar(float v) {
    return static_cast<_Float16>(v);
  }
};

// A chunk is E consecutive elements handled by one lane: E = 8 whenever a
// 16-bit type is involved (one 16-byte vector of it), else 4.  A chunk of a
// wider type spans E * sizeof(T) / 16 vectors.
template <typename T, int E, bool STREAM = true>
__device__ __forceinline__ void load_chunk(const T *p, float *f) {
  constexpr int NV = E * (int)sizeof(T) / 16;
  static_assert(NV >= 1, "chunk smaller than one vector");
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    u32x4 r = STREAM ? ld16_stream(p + v * io<T>::EPV)
                     : ld16_cached(p + v * io<T>::EPV);
    io<T>::unpack(r, f + v * io<T>::EPV);
  }
}

template <typename T, int E>
__device__ __forceinline__ void store_chunk(T *p, const float *f) {
  constexpr int NV = E * (int)sizeof(T) / 16;
#pragma unroll
  for (int v = 0; v < NV; ++v)
    st16_stream(p + v * io<T>::EPV, io<T>::pack(f + v * io<T>::EPV));
}

// Stores a chunk (p may be null: nothing is written) and replaces f by the
// values as stored, taken from the very registers that were written.  Code
// that accumulates "the tensor as stored" must go through this: rounding f a
// second time in a separate expression can differ in the last place, because
// the compiler may fuse the arithmetic that produced f into one of the two
// conversions (a mixed-precision fma rounds once, a product followed by a
// conversion rounds twice).
template <typename T, int E>
__device__ __forceinline__ void store_chunk_readback(T *p, float *f) {
  constexpr int NV = E * (int)sizeof(T) / 16;
  static_assert(NV >= 1, "chunk smaller than one vector");
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const u32x4 r = io<T>::pack(f + v * io<T>::EPV);
    if (p != nullptr) st16_stream(p + v * io<T>::EPV, r);
    io<T>::unpack(r, f + v * io<T>::EPV);
  }
}

// A chunk kept in its packed storage form, for loads issued one iteration
// ahead of their use (software prefetch): E * sizeof(T) / 4 registers.
template <typename T, int E> struct RawChunk {
  static constexpr int NV = E * (int)sizeof(T) / 16;
  u32x4 r[NV];
  __device__ __forceinline__ void load(const T *p) {
#pragma unroll
    for (int v = 0; v < NV; ++v) r[v] = ld16_stream(p + v * io<T>::EPV);
  }
  __device__ __forceinline__ void load_cached(const T *p) {
#pragma unroll
    for (int v = 0; v < NV; ++v) r[v] = ld16_cached(p + v * io<T>::EPV);
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int v = 0; v < NV; ++v) r[v] = u32x4{0u, 0u, 0u, 0u};
  }
  __device__ __forceinline__ void unpack(float *f) const {
#pragma unroll
    for (int v = 0; v < NV; ++v) io<T>::unpack(r[v], f + v * io<T>::EPV);
  }
};

template <typename A, typename B> struct chunk_elems {
  static constexpr int value =
      16 / (int)(sizeof(A) < sizeof(B) ? sizeof(A) : sizeof(B));
};

// ---------------------------------------------------------------------------
// wave64 reductions.  Four DPP steps make every row of 16 lanes uniform
// (quad swaps, then the half-row and row mirrors); the four row values are
// then read through v_readlane and combined in a fixed order, so every lane
// ends with the same, deterministic result.  All 64 lanes must be active.
// ---------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}

constexpr int kDppQuadSwap1 = 0xB1;     // quad_perm:[1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;     // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

__device__ __forceinline__ float readlane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

struct OpSum {
  static __device__ __forceinline__ float apply(float a, float b) {
    return a + b;
  }
};
struct OpMax {
  static __device__ __forceinline__ float apply(float a, float b) {
    return fmaxf(a, b);
  }
};

template <typename Op> __device__ __forceinline__ float wave_allreduce(float v) {
  v = Op::apply(v, dpp_mov<kDppQuadSwap1>(v));
  v = Op::apply(v, dpp_mov<kDppQuadSwap2>(v));
  v = Op::apply(v, dpp_mov<kDppRowHalfMirror>(v));
  v = Op::apply(v, dpp_mov<kDppRowMirror>(v));
  float r0 = readlane(v, 0), r1 = readlane(v, 16);
  float r2 = readlane(v, 32), r3 = readlane(v, 48);
  return Op::apply(Op::apply(r0, r1), Op::apply(r2, r3));
}
__device__ __forceinline__ float wave_sum(float v) {
  return wave_allreduce<OpSum>(v);
}
__device__ __forceinline__ float wave_max(float v) {
  return wave_allreduce<OpMax>(v);
}

// Welford partial statistics of a set of values: count, mean, and the sum of
// squared deviations from that mean.  chan_merge combines two disjoint sets
// (Chan, Golub, LeVeque 1979), as cuChanOnlineSum does in the reference
// (oslo/torch/_C/csrc/fused_layer_norm.cu:22-38).
struct Welford {
  float n, mean, m2;
};

__device__ __forceinline__ Welford chan_merge(Welford a, Welford b) {
  const float n = a.n + b.n;
  const float r = n > 0.f ? b.n * __builtin_amdgcn_rcpf(n) : 0.f;
  const float d = b.mean - a.mean;
  Welford o;
  o.n = n;
  o.mean = a.mean + d * r;
  o.m2 = a.m2 + b.m2 + d * d * (a.n * r);
  return o;
}

template <int CTRL> __device__ __forceinline__ Welford dpp_welford(Welford v) {
  Welford o;
  o.n = dpp_mov<CTRL>(v.n);
  o.mean = dpp_mov<CTRL>(v.mean);
  o.m2 = dpp_mov<CTRL>(v.m2);
  return o;
}

// All-reduce of Welford partials over the wave: four DPP butterfly steps
// inside each row of 16 lanes, then the four row results (read from lanes 0,
// 16, 32, 48) are merged in a fixed order, so every lane returns the same bits.
__device__ __forceinline__ Welford wave_welford(Welford v) {
  v = chan_merge(v, dpp_welford<kDppQuadSwap1>(v));
  v = chan_merge(v, dpp_welford<kDppQuadSwap2>(v));
  v = chan_merge(v, dpp_welford<kDppRowHalfMirror>(v));
  v = chan_merge(v, dpp_welford<kDppRowMirror>(v));
  Welford r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i].n = readlane(v.n, 16 * i);
    r[i].mean = readlane(v.mean, 16 * i);
    r[i].m2 = readlane(v.m2, 16 * i);
  }
  return chan_merge(chan_merge(r[0], r[1]), chan_merge(r[2], r[3]));
}

// The same all-reduce when every lane holds the same number of values
// (`per_lane`): the merge of two equal-sized sets needs no division and is
// symmetric, mean = (ma + mb) / 2, M2 = M2a + M2b + (mb - ma)^2 * n / 2.
__device__ __forceinline__ void merge_equal(float &mean, float &m2, float omean,
                                            float om2, float n_each) {
  const float d = omean - mean;
  mean = 0.5f * (mean + omean);
  m2 = (m2 + om2) + d * d * (0.5f * n_each);
}

__device__ __forceinline__ Welford wave_welford_equal(float mean, float m2,
                                                      float per_lane) {
  merge_equal(mean, m2, dpp_mov<kDppQuadSwap1>(mean),
              dpp_mov<kDppQuadSwap1>(m2), per_lane);
  merge_equal(mean, m2, dpp_mov<kDppQuadSwap2>(mean),
              dpp_mov<kDppQuadSwap2>(m2), 2.f * per_lane);
  merge_equal(mean, m2, dpp_mov<kDppRowHalfMirror>(mean),
              dpp_mov<kDppRowHalfMirror>(m2), 4.f * per_lane);
  merge_equal(mean, m2, dpp_mov<kDppRowMirror>(mean),
              dpp_mov<kDppRowMirror>(m2), 8.f * per_lane);
  float ma = readlane(mean, 0), qa = readlane(m2, 0);
  float mb = readlane(mean, 32), qb = readlane(m2, 32);
  merge_equal(ma, qa, readlane(mean, 16), readlane(m2, 16), 16.f * per_lane);
  merge_equal(mb, qb, readlane(mean, 48), readlane(m2, 48), 16.f * per_lane);
  merge_equal(ma, qa, mb, qb, 32.f * per_lane);
  Welford w;
  w.n = 64.f * per_lane;
  w.mean = ma;
  w.m2 = qa;
  return w;
}

// 1 / sqrt(a): hardware estimate plus one Newton step (error below 1 ulp).
__device__ __forceinline__ float rsqrt_refined(float a) {
  float y = __builtin_amdgcn_rsqf(a);
  const float h = 0.5f * a * y;
  const float r = fmaf(y, 0.5f - h * y, y);
  // a = inf gives 0 and a = 0 gives inf, as rsqrt does; the Newton step would
  // turn both into NaN (inf * 0)
  return a > 0.f && a < __builtin_inff() ? r : y;
}

// Reduction of the values held by lanes 0..15 (one DPP row), returned to every
// lane through lane 0.  Used to combine the per-wave results of the up to 16
// waves that share a row: lane l < wpr reads wave l's value from LDS, the
// other lanes pass the identity.
template <typename Op> __device__ __forceinline__ float row16_allreduce(float v) {
  v = Op::apply(v, dpp_mov<kDppQuadSwap1>(v));
  v = Op::apply(v, dpp_mov<kDppQuadSwap2>(v));
  v = Op::apply(v, dpp_mov<kDppRowHalfMirror>(v));
  v = Op::apply(v, dpp_mov<kDppRowMirror>(v));
  return readlane(v, 0);
}

// A product / difference that is rounded on its own and never fused with a
// neighbouring operation into a multiply-add.  Two kernels that must
// reproduce the same bits (a forward pass and the backward pass that
// recomputes it) cannot leave that choice to the optimiser; the header's
// __fmul_rn / __fsub_rn are plain operators here and do get fused.
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// The value as it sits in a 32-bit register, hidden from the optimiser.  A
// second output that must be a conversion of the float32 result *as stored*
// (the 16-bit copy of a float32 master weight) goes through this: otherwise
// the conversion may be fused with the multiply-add that produced the value
// and round the unrounded result once, which differs from converting the
// stored float32 value whenever that lies on a 16-bit rounding tie.
__device__ __forceinline__ float pinned(float v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Reduction within each group of LPR (8, 16 or 32) consecutive lanes; every
// lane of a group receives its group's result (each step is symmetric, so the
// lanes of a group hold the same bits).
template <typename Op, int LPR>
__device__ __forceinline__ float group_allreduce(float v) {
  static_assert(LPR == 8 || LPR == 16 || LPR == 32, "group size");
  v = Op::apply(v, dpp_mov<kDppQuadSwap1>(v));
  v = Op::apply(v, dpp_mov<kDppQuadSwap2>(v));
  v = Op::apply(v, dpp_mov<kDppRowHalfMirror>(v));
  if constexpr (LPR >= 16) v = Op::apply(v, dpp_mov<kDppRowMirror>(v));
  if constexpr (LPR >= 32) v = Op::apply(v, __shfl_xor(v, 16));
  return v;
}

// Reduction over the WPR consecutive waves that share one row.  `red` is LDS
// scratch of at least (waves in block) floats, `slot` selects one of two such
// areas so that back-to-back reductions need only one barrier each.
template <typename Op, int WPR>
__device__ __forceinline__ float row_allreduce(float v, float *red, int wave,
                                               int lane) {
  v = wave_allreduce<Op>(v);
  if constexpr (WPR > 1) {
    if (lane == 0) red[wave] = v;
    __syncthreads();
    const int first = wave - (wave % WPR);
    float r = red[first];
#pragma unroll
    for (int w = 1; w < WPR; ++w) r = Op::apply(r, red[first + w]);
    v = r;
  }
  return v;
}

// ---------------------------------------------------------------------------
// Philox4x32-10 (Salmon et al., SC'11; the constants of Random123 and of
// ATen/core/PhiloxRNGEngine.h).
// ---------------------------------------------------------------------------
struct Philox4 {
  uint32_t x, y, z, w;
};

// a ^ b ^ c: one v_bitop3_b32 (truth table 0x96) on the GPU
__device__ __host__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
#else
  return a ^ b ^ c;
#endif
}

__device__ __host__ __forceinline__ Philox4 philox4x32_10(uint32_t c0,
                                                           uint32_t c1,
                                                           uint32_t c2,
                                                           uint32_t c3,
                                                           uint32_t k0,
                                                           uint32_t k1) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  constexpr uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)M0 * c0;
    const uint64_t p1 = (uint64_t)M1 * c2;
    const uint32_t n0 = xor3((uint32_t)(p1 >> 32), c1, k0);
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = xor3((uint32_t)(p0 >> 32), c3, k1);
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0;
    c1 = n1;
    c2 = n2;
    c3 = n3;
    k0 += W0;
    k1 += W1;
  }
  return Philox4{c0, c1, c2, c3};
}

// Keep decisions of the 8 elements of one dropout group (see oslo_hip.h):
// bit e of the result is set when element e of the group is kept.
__device__ __host__ __forceinline__ uint32_t
dropout_keep_bits(uint64_t group, uint64_t seed, uint64_t offset,
                  uint32_t threshold) {
  const Philox4 r =
      philox4x32_10((uint32_t)offset, (uint32_t)(offset >> 32),
                    (uint32_t)group, (uint32_t)(group >> 32), (uint32_t)seed,
                    (uint32_t)(seed >> 32));
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  uint32_t bits = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bits |= ((w[i] & 0xffffu) >= threshold ? 1u : 0u) << (2 * i);
    bits |= ((w[i] >> 16) >= threshold ? 1u : 0u) << (2 * i + 1);
  }
  return bits;
}

// Dropout parameters of one call.  Element i of the flattened tensor belongs
// to group i >> 3 and is kept when bit i & 7 of that group's keep bits is set.
struct DropArgs {
  uint64_t seed, offset;
  uint32_t threshold;  // keep when the 16-bit draw >= threshold
  float scale;         // 1 / (1 - p), 0 when p >= 1
  // non-null: {seed, offset} are read from device memory when the kernel
  // runs (seed = dev[0], offset = dev[1] + offset), so that a launch captured
  // in a graph draws a new mask on every replay
  const uint64_t *dev;
};

// The (seed, offset) pair a kernel works with; uniform over the launch.
__device__ __forceinline__ DropArgs resolve_drop(DropArgs d) {
  if (d.dev != nullptr) {
    d.seed = d.dev[0];
    d.offset += d.dev[1];
  }
  return d;
}

__device__ __host__ __forceinline__ bool keep_element(int64_t i, const DropArgs &d) {
  const uint32_t bits =
      dropout_keep_bits((uint64_t)i >> 3, d.seed, d.offset, d.threshold);
  return (bits >> (i & 7)) & 1u;
}

static inline DropArgs make_drop(float p, uint64_t seed, uint64_t offset) {
  DropArgs d;
  d.seed = seed;
  d.offset = offset;
  d.dev = current_rng_state();  // set by the *_rng entry points, else null
  double t = (double)p * 65536.0 + 0.5;
  d.threshold = t >= 65536.0 ? 65536u : (uint32_t)t;
  d.scale = p < 1.0f ? 1.0f / (1.0f - p) : 0.f;
  return d;
}

// Keep bits of the E elements of chunk c of `row` (dropout on the flattened
// [rows, row_length] tensor: element i belongs to group i >> 3).  A 4-element chunk
// takes the low or the high half of its group's eight bits.
template <int E>
__device__ __forceinline__ uint32_t chunk_keep_bits(int64_t row, int row_length, int c,
                                                    const DropArgs &d) {
  const uint64_t flat = (uint64_t)row * (uint64_t)row_length + (uint64_t)c * E;
  uint32_t keep = dropout_keep_bits(flat >> 3, d.seed, d.offset, d.threshold);
  if constexpr (E == 4) keep >>= (uint32_t)(flat & 4u);
  return keep;
}

// The same keep decisions straight from the generator's words, for kernels
// that use every decision once: element e of the chunk is kept when 16-bit
// field (e & 1) of word w[e >> 1] reaches the threshold.  Comparing a field
// where it is used (one sub-word compare and one select) takes fewer
// instructions than packing the decisions into bits and testing the bits again.
template <int E>
struct KeepWords {
  uint32_t w[E / 2];
  uint32_t threshold;
  __device__ __host__ __forceinline__ bool kept(int e) const {
    const uint32_t f = (e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu);
    return f >= threshold;
  }
};

template <int E>
__device__ __host__ __forceinline__ KeepWords<E>
group_keep_words(uint64_t flat, uint64_t seed, uint64_t offset, uint32_t threshold) {
  static_assert(E == 4 || E == 8, "a chunk is a dropout group or half of one");
  const uint64_t group = flat >> 3;
  const Philox4 r =
      philox4x32_10((uint32_t)offset, (uint32_t)(offset >> 32),
                    (uint32_t)group, (uint32_t)(group >> 32), (uint32_t)seed,
                    (uint32_t)(seed >> 32));
  KeepWords<E> k;
  k.threshold = threshold;
  if constexpr (E == 8) {
    k.w[0] = r.x;
    k.w[1] = r.y;
    k.w[2] = r.z;
    k.w[3] = r.w;
  } else {
    const bool hi = (flat & 4u) != 0u;  // which half of the group the chunk is
    k.w[0] = hi ? r.z : r.x;
    k.w[1] = hi ? r.w : r.y;
  }
  return k;
}

template <int E>
__device__ __forceinline__ KeepWords<E> chunk_keep_words(int64_t row, int row_length, int c,
                                                         const DropArgs &d) {
  const uint64_t flat = (uint64_t)row * (uint64_t)row_length + (uint64_t)c * E;
  return group_keep_words<E>(flat, d.seed, d.offset, d.threshold);
}

}  // namespace oslo
