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
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
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

}  // namespace oslo
