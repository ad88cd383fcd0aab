// Device-side element codecs: run-time typed, vectorised loads into a compute type and stores
// out of it.  The element type is a kernel argument (wave-uniform), so each `switch` below is a
// scalar branch; the loads and stores inside each arm are full-width vector accesses.
//
// Encoding rules follow the reference's write path (nx/lib/nx/shared.ex:136-194,
// nx/lib/nx/floating.ex:60-64, nx/lib/nx/type.ex:128-158): integers wrap to the low bits,
// f32/f16 round to nearest even, bf16 is the f32 encoding with the low 16 bits dropped, and a
// NaN is always written as the canonical quiet NaN of the output type.
#pragma once
#ifndef __HIPCC_RTC__  // the run-time compiler has the device runtime built in and is given headers by name
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hipnx.h"
#else
#include "hipnx.h"
#endif

namespace hipnx {

typedef _Float16 f16_t;

template <int BYTES>
struct alignas(BYTES) raw_vec {
  unsigned char b[BYTES];
};

// ---- scalar decode ------------------------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// ---- scalar encode ------------------------------------------------------------------------

__device__ __forceinline__ uint16_t f32_to_bf16_bits_trunc(float f) {
  uint32_t b = __float_as_uint(f);
  return (f != f) ? (uint16_t)0x7FC0 : (uint16_t)(b >> 16);
}
// round-to-nearest-even to bf16 (the HIPNX_BF16_RNE output code)
__device__ __forceinline__ uint16_t f32_to_bf16_bits_rne(float f) {
  uint32_t b = __float_as_uint(f);
  return (f != f) ? (uint16_t)0x7FC0 : (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ uint32_t f32_canon_bits(float f) { return (f != f) ? 0x7FC00000u : __float_as_uint(f); }
__device__ __forceinline__ uint64_t f64_canon_bits(double d) {
  return (d != d) ? 0x7FF8000000000000ull : (uint64_t)__double_as_longlong(d);
}
__device__ __forceinline__ uint16_t f16_bits(f16_t h) {
  union { f16_t h; uint16_t u; } x;
  x.h = h;
  return x.u;
}
__device__ __forceinline__ f16_t bits_f16(uint16_t u) {
  union { f16_t h; uint16_t u; } x;
  x.u = u;
  return x.h;
}
// The conversion is kept apart from the arithmetic that made `f` (the empty asm): the compiler otherwise turns a product
// followed by this rounding into one mixed-precision fma with +0 as the addend, and (-x) * 0 = -0 comes out as +0.
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  asm("" : "+v"(f));
  return (f != f) ? (uint16_t)0x7E00 : f16_bits((f16_t)f);
}
// f64 -> f32 with round-to-odd, so that a following round-to-nearest narrowing equals a single
// rounding of the f64 value
__device__ __forceinline__ float f64_to_f32_round_odd(double d) {
  float f = __double2float_rz(d);
  uint32_t b = __float_as_uint(f);
  if ((double)f != d && (b & 0x7F800000u) != 0x7F800000u) b |= 1u;
  return __uint_as_float(b);
}
// one rounding of the f64 value: round-to-odd keeps 24 significant bits, more than the 8 + 2 that make
// the second rounding exact
__device__ __forceinline__ uint16_t f64_to_bf16_bits_rne(double d) { return f32_to_bf16_bits_rne(f64_to_f32_round_odd(d)); }
__device__ __forceinline__ uint16_t f64_to_f16_bits(double d) {
  return (d != d) ? (uint16_t)0x7E00 : f16_bits((f16_t)f64_to_f32_round_odd(d));
}

// ---- compute-type traits ------------------------------------------------------------------

template <typename CT>
struct conv;

template <>
struct conv<float> {
  template <typename S> static __device__ __forceinline__ float from_int(S v) { return (float)v; }
  static __device__ __forceinline__ float from_f64(double v) { return (float)v; }
  static __device__ __forceinline__ float from_f32(float v) { return v; }
  static __device__ __forceinline__ uint16_t to_bf16(float v) { return f32_to_bf16_bits_trunc(v); }
  static __device__ __forceinline__ uint16_t to_bf16_rne(float v) { return f32_to_bf16_bits_rne(v); }
  static __device__ __forceinline__ uint16_t to_f16(float v) { return f32_to_f16_bits(v); }
  static __device__ __forceinline__ uint32_t to_f32(float v) { return f32_canon_bits(v); }
  static __device__ __forceinline__ uint64_t to_f64(float v) { return f64_canon_bits((double)v); }
  // float -> integer only happens for 0/1 predicate results and whole numbers in range
  static __device__ __forceinline__ int64_t to_int(float v) { return (int64_t)v; }
};
template <>
struct conv<double> {
  template <typename S> static __device__ __forceinline__ double from_int(S v) { return (double)v; }
  static __device__ __forceinline__ double from_f64(double v) { return v; }
  static __device__ __forceinline__ double from_f32(float v) { return (double)v; }
  static __device__ __forceinline__ uint16_t to_bf16(double v) { return f32_to_bf16_bits_trunc((float)v); }
  static __device__ __forceinline__ uint16_t to_bf16_rne(double v) { return f64_to_bf16_bits_rne(v); }
  static __device__ __forceinline__ uint16_t to_f16(double v) { return f64_to_f16_bits(v); }
  static __device__ __forceinline__ uint32_t to_f32(double v) { return f32_canon_bits((float)v); }
  static __device__ __forceinline__ uint64_t to_f64(double v) { return f64_canon_bits(v); }
  static __device__ __forceinline__ int64_t to_int(double v) { return (int64_t)v; }
};
template <>
struct conv<int64_t> {  // also carries u64 bit patterns
  template <typename S> static __device__ __forceinline__ int64_t from_int(S v) { return (int64_t)v; }
  static __device__ __forceinline__ int64_t from_f64(double v) { return (int64_t)v; }
  static __device__ __forceinline__ int64_t from_f32(float v) { return (int64_t)v; }
  static __device__ __forceinline__ uint16_t to_bf16(int64_t v) { return f32_to_bf16_bits_trunc((float)(double)v); }
  static __device__ __forceinline__ uint16_t to_bf16_rne(int64_t v) { return f64_to_bf16_bits_rne((double)v); }
  static __device__ __forceinline__ uint16_t to_f16(int64_t v) { return f64_to_f16_bits((double)v); }
  static __device__ __forceinline__ uint32_t to_f32(int64_t v) { return __float_as_uint((float)(double)v); }
  static __device__ __forceinline__ uint64_t to_f64(int64_t v) { return (uint64_t)__double_as_longlong((double)v); }
  static __device__ __forceinline__ int64_t to_int(int64_t v) { return v; }
};

// ---- vector load: E consecutive elements of run-time type `dt` starting at element `idx` ---
// `idx` must be a multiple of E when E > 1 (the caller guarantees 16-byte-or-element alignment).

// ALIGNED = false: `idx` is any element (the bytes are fetched through a copy whose source claims no alignment, which
// the compiler still turns into whole-vector loads: global memory takes them at any address).
// (Written into its destination, not returned: with the bytes returned by value the compiler took an f32 -> bf16
// conversion's two 16-byte loads apart into sixteen 2-byte ones.)
// NT: the access carries the non-temporal hint -- for tensors far larger than the last-level cache, which then keeps
// less of what will not be read again before it is evicted anyway: a 1 GiB copy 6.16 -> 6.50 TB/s, x + y of 1 GiB a
// side 6.02 -> 6.43 TB/s.  A template parameter all the way down: a run-time flag leaves a hinted and a plain access
// on two branches, which the compiler merges into one without the hint.
typedef uint32_t __attribute__((ext_vector_type(4))) raw_u4;
typedef uint32_t __attribute__((ext_vector_type(2))) raw_u2;
template <int N, bool ALIGNED, bool NT = false>
__device__ __forceinline__ void fetch_raw(raw_vec<N> *dst, const void *q) {
  if constexpr (NT && ALIGNED && N == 16) {
    const raw_u4 w = __builtin_nontemporal_load(reinterpret_cast<const raw_u4 *>(q));
    __builtin_memcpy(dst, &w, 16);
  } else if constexpr (NT && ALIGNED && N == 8) {
    const raw_u2 w = __builtin_nontemporal_load(reinterpret_cast<const raw_u2 *>(q));
    __builtin_memcpy(dst, &w, 8);
  } else if constexpr (ALIGNED) {
    *dst = *reinterpret_cast<const raw_vec<N> *>(q);
  } else {
    __builtin_memcpy(dst, q, N);
  }
}
template <int N, bool NT = false>
__device__ __forceinline__ void put_raw(void *q, const raw_vec<N> &src) {
  if constexpr (NT && N == 16) {
    raw_u4 w;
    __builtin_memcpy(&w, &src, 16);
    __builtin_nontemporal_store(w, reinterpret_cast<raw_u4 *>(q));
  } else if constexpr (NT && N == 8) {
    raw_u2 w;
    __builtin_memcpy(&w, &src, 8);
    __builtin_nontemporal_store(w, reinterpret_cast<raw_u2 *>(q));
  } else {
    *reinterpret_cast<raw_vec<N> *>(q) = src;
  }
}

template <typename CT, int E, bool ALIGNED = true, bool NT = false>
__device__ __forceinline__ void load_vec(const void *__restrict__ p, int dt, int64_t idx, CT (&v)[E]) {
  switch (dt) {
    case HIPNX_U8: {
      raw_vec<E> r;
      fetch_raw<E, ALIGNED, NT>(&r, (const uint8_t *)p + idx);
#pragma unroll
      for (int i = 0; i < E; i++) v[i] = conv<CT>::from_int((uint32_t)r.b[i]);
      break;
    }
    case HIPNX_S8: {
      raw_vec<E> r;
      fetch_raw<E, ALIGNED, NT>(&r, (const uint8_t *)p + idx);
#pragma unroll
      for (int i = 0; i < E; i++) v[i] = conv<CT>::from_int((int32_t)(int8_t)r.b[i]);
      break;
    }
    case HIPNX_U16:
    case HIPNX_S16:
    case HIPNX_F16:
    case HIPNX_BF16: {
      raw_vec<2 * E> r;
      fetch_raw<2 * E, ALIGNED, NT>(&r, (const uint16_t *)p + idx);
      const uint16_t *h = reinterpret_cast<const uint16_t *>(r.b);
#pragma unroll
      for (int i = 0; i < E; i++) {
        if (dt == HIPNX_U16) v[i] = conv<CT>::from_int((uint32_t)h[i]);
        else if (dt == HIPNX_S16) v[i] = conv<CT>::from_int((int32_t)(int16_t)h[i]);
        else if (dt == HIPNX_F16) v[i] = conv<CT>::from_f32((float)bits_f16(h[i]));
        else v[i] = conv<CT>::from_f32(bf16_bits_to_f32(h[i]));
      }
      break;
    }
    case HIPNX_U32:
    case HIPNX_S32:
    case HIPNX_F32: {
      constexpr int B = 4 * E, CH = B > 16 ? 16 : B;
      uint32_t w[E];
#pragma unroll
      for (int c = 0; c < B / CH; c++)
        fetch_raw<CH, ALIGNED, NT>(reinterpret_cast<raw_vec<CH> *>(&w[c * CH / 4]), (const char *)p + idx * 4 + c * CH);
#pragma unroll
      for (int i = 0; i < E; i++) {
        if (dt == HIPNX_U32) v[i] = conv<CT>::from_int(w[i]);
        else if (dt == HIPNX_S32) v[i] = conv<CT>::from_int((int32_t)w[i]);
        else v[i] = conv<CT>::from_f32(__uint_as_float(w[i]));
      }
      break;
    }
    default: {  // U64, S64, F64
      constexpr int B = 8 * E, CH = B > 16 ? 16 : B;
      uint64_t w[E];
#pragma unroll
      for (int c = 0; c < B / CH; c++)
        fetch_raw<CH, ALIGNED, NT>(reinterpret_cast<raw_vec<CH> *>(reinterpret_cast<char *>(w) + c * CH), (const char *)p + idx * 8 + c * CH);
#pragma unroll
      for (int i = 0; i < E; i++) {
        if (dt == HIPNX_F64) v[i] = conv<CT>::from_f64(__longlong_as_double((long long)w[i]));
        else if (dt == HIPNX_U64) v[i] = conv<CT>::from_int((uint64_t)w[i]);
        else v[i] = conv<CT>::from_int((int64_t)w[i]);
      }
      break;
    }
  }
}

template <typename CT>
__device__ __forceinline__ CT load_one(const void *__restrict__ p, int dt, int64_t idx) {
  CT v[1];
  load_vec<CT, 1>(p, dt, idx, v);
  return v[0];
}

template <typename CT, int E, bool NT = false>
__device__ __forceinline__ void store_vec(void *__restrict__ p, int dt, int64_t idx, const CT (&v)[E]) {
  switch (dt) {
    case HIPNX_U8:
    case HIPNX_S8: {
      raw_vec<E> r;
#pragma unroll
      for (int i = 0; i < E; i++) r.b[i] = (unsigned char)conv<CT>::to_int(v[i]);
      put_raw<E, NT>((uint8_t *)p + idx, r);
      break;
    }
    case HIPNX_U16:
    case HIPNX_S16:
    case HIPNX_F16:
    case HIPNX_BF16:
    case HIPNX_BF16_RNE: {
      raw_vec<2 * E> r;
      uint16_t *h = reinterpret_cast<uint16_t *>(r.b);
#pragma unroll
      for (int i = 0; i < E; i++) {
        if (dt == HIPNX_F16) h[i] = conv<CT>::to_f16(v[i]);
        else if (dt == HIPNX_BF16) h[i] = conv<CT>::to_bf16(v[i]);
        else if (dt == HIPNX_BF16_RNE) h[i] = conv<CT>::to_bf16_rne(v[i]);
        else h[i] = (uint16_t)conv<CT>::to_int(v[i]);
      }
      put_raw<2 * E, NT>((uint16_t *)p + idx, r);
      break;
    }
    case HIPNX_U32:
    case HIPNX_S32:
    case HIPNX_F32: {
      constexpr int B = 4 * E, CH = B > 16 ? 16 : B;
      uint32_t w[E];
#pragma unroll
      for (int i = 0; i < E; i++) w[i] = dt == HIPNX_F32 ? conv<CT>::to_f32(v[i]) : (uint32_t)conv<CT>::to_int(v[i]);
#pragma unroll
      for (int c = 0; c < B / CH; c++)
        put_raw<CH, NT>((char *)p + idx * 4 + c * CH, *reinterpret_cast<const raw_vec<CH> *>(&w[c * CH / 4]));
      break;
    }
    default: {
      constexpr int B = 8 * E, CH = B > 16 ? 16 : B;
      uint64_t w[E];
#pragma unroll
      for (int i = 0; i < E; i++) w[i] = dt == HIPNX_F64 ? conv<CT>::to_f64(v[i]) : (uint64_t)conv<CT>::to_int(v[i]);
#pragma unroll
      for (int c = 0; c < B / CH; c++)
        put_raw<CH, NT>((char *)p + idx * 8 + c * CH, *reinterpret_cast<const raw_vec<CH> *>(reinterpret_cast<const char *>(w) + c * CH));
      break;
    }
  }
}

template <typename CT>
__device__ __forceinline__ void store_one(void *__restrict__ p, int dt, int64_t idx, CT x) {
  CT v[1] = {x};
  store_vec<CT, 1>(p, dt, idx, v);
}

}  // namespace hipnx
