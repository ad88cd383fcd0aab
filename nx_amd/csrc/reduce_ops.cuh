// Reducer policies shared by the reduction kernels and the fused element-wise + row-reduction kernel:
// what an accumulator is, how an element is folded in, how two accumulators combine, and how the
// result is stored.  The kernels that use them fix the order of the folds; two kernels that walk a
// row in the same order with the same policy give the same bits.
#pragma once
#ifndef __HIPCC_RTC__
#include <type_traits>
#include <utility>
#endif

#include "dtypes.cuh"

namespace hipnx {

constexpr int E = 8;
constexpr int BLOCK = 256;
constexpr int WAVE = 64;

// ---- reducer policies -----------------------------------------------------------------------

template <typename CT, int OP, bool UNS>
struct PlainReducer {
  typedef CT acc_t;
  // whether the result is the same bits whichever elements a lane is given (sums and products of floats are not:
  // their order of additions is part of the result)
  static constexpr bool any_order = OP != HIPNX_RED_SUM && OP != HIPNX_RED_PRODUCT;
  static __device__ __forceinline__ acc_t init() {
    if constexpr (OP == HIPNX_RED_SUM || OP == HIPNX_RED_ANY) return (CT)0;
    else if constexpr (OP == HIPNX_RED_PRODUCT || OP == HIPNX_RED_ALL) return (CT)1;
    else if constexpr (std::is_floating_point<CT>::value) return OP == HIPNX_RED_MAX ? (CT)-INFINITY : (CT)INFINITY;
    else if constexpr (UNS) return OP == HIPNX_RED_MAX ? (int64_t)0 : (int64_t)-1;
    else return OP == HIPNX_RED_MAX ? INT64_MIN : INT64_MAX;
  }
  static __device__ __forceinline__ acc_t combine(acc_t a, acc_t b) {
    // all / any work on truth values 0 / 1 (see accumulate)
    if constexpr (OP == HIPNX_RED_ALL) return (a != (CT)0 && b != (CT)0) ? (CT)1 : (CT)0;
    else if constexpr (OP == HIPNX_RED_ANY) return (a != (CT)0 || b != (CT)0) ? (CT)1 : (CT)0;
    else if constexpr (std::is_floating_point<CT>::value) {
      if constexpr (OP == HIPNX_RED_SUM) return a + b;
      else if constexpr (OP == HIPNX_RED_PRODUCT) return a * b;
      else if constexpr (OP == HIPNX_RED_MAX) return (a != a || b != b) ? (CT)NAN : (b > a ? b : a);
      else return (a != a || b != b) ? (CT)NAN : (b < a ? b : a);
    } else {
      if constexpr (OP == HIPNX_RED_SUM) return (int64_t)((uint64_t)a + (uint64_t)b);
      else if constexpr (OP == HIPNX_RED_PRODUCT) return (int64_t)((uint64_t)a * (uint64_t)b);
      else if constexpr (UNS) {
        if constexpr (OP == HIPNX_RED_MAX) return (uint64_t)b > (uint64_t)a ? b : a;
        else return (uint64_t)b < (uint64_t)a ? b : a;
      } else {
        if constexpr (OP == HIPNX_RED_MAX) return b > a ? b : a;
        else return b < a ? b : a;
      }
    }
  }
  static __device__ __forceinline__ acc_t seed(acc_t a, int64_t) { return a; }
  // (for all / any an element counts as true unless it equals 0 -- NaN included,
  // binary_backend.ex:1293-1314)
  static __device__ __forceinline__ acc_t accumulate(acc_t a, CT x, int64_t) { return combine(a, x); }
  static __device__ __forceinline__ acc_t shfl_xor(acc_t a, int m) { return __shfl_xor(a, m, WAVE); }
};

template <typename CT>
struct ArgAcc {
  CT v;
  int i;  // position along the reduced axis (extents below 2^31); -1 = empty
};

template <typename CT, int OP, int TIE, bool UNS>
struct ArgReducer {
  typedef ArgAcc<CT> acc_t;
  static constexpr bool any_order = true;  // (a lane must still meet its own elements in rising order)
  static constexpr bool FP = std::is_floating_point<CT>::value;
  // the worst possible value: nothing is worse, so a lane seeded with {worst, first index} is
  // already the right answer for "no better element seen yet"
  static __device__ __forceinline__ acc_t init() {
    if constexpr (FP) return acc_t{OP == HIPNX_ARGMAX ? (CT)-INFINITY : (CT)INFINITY, -1};
    else if constexpr (UNS) return acc_t{OP == HIPNX_ARGMAX ? (CT)0 : (CT)-1, -1};
    else return acc_t{OP == HIPNX_ARGMAX ? (CT)INT64_MIN : (CT)INT64_MAX, -1};
  }
  static __device__ __forceinline__ acc_t seed(acc_t a, int64_t first) { a.i = (int)first; return a; }
  static __device__ __forceinline__ bool better(CT x, CT y) {  // x strictly better than y
    if constexpr (std::is_same<CT, int64_t>::value && UNS)
      return OP == HIPNX_ARGMAX ? (uint64_t)x > (uint64_t)y : (uint64_t)x < (uint64_t)y;
    else return OP == HIPNX_ARGMAX ? x > y : x < y;
  }
  static __device__ __forceinline__ bool better_or_equal(CT x, CT y) {
    if constexpr (std::is_same<CT, int64_t>::value && UNS)
      return OP == HIPNX_ARGMAX ? (uint64_t)x >= (uint64_t)y : (uint64_t)x <= (uint64_t)y;
    else return OP == HIPNX_ARGMAX ? x >= y : x <= y;
  }
  // any order (cross-lane tree, partials): NaN beats numbers, the larger index wins among NaNs
  static __device__ __forceinline__ acc_t combine(acc_t a, acc_t b) {
    if (b.i < 0) return a;
    if (a.i < 0) return b;
    if constexpr (FP) {
      const bool an = a.v != a.v, bn = b.v != b.v;
      if (an | bn) {
        if (an && bn) return a.i > b.i ? a : b;
        return an ? a : b;
      }
    }
    if (better(b.v, a.v)) return b;
    if (better(a.v, b.v)) return a;
    if constexpr (TIE == HIPNX_TIE_LOW) return a.i < b.i ? a : b;
    else return a.i > b.i ? a : b;
  }
  // streaming step of a seeded lane: indices only grow, so a tie resolves by position, and a
  // NaN extreme is sticky by itself (every comparison with it is false)
  static __device__ __forceinline__ acc_t accumulate(acc_t a, CT x, int64_t idx) {
    bool take = TIE == HIPNX_TIE_LOW ? better(x, a.v) : better_or_equal(x, a.v);
    if constexpr (FP) take |= x != x;
    return take ? acc_t{x, (int)idx} : a;
  }
  static __device__ __forceinline__ acc_t shfl_xor(acc_t a, int m) {
    acc_t r;
    r.v = __shfl_xor(a.v, m, WAVE);
    r.i = __shfl_xor(a.i, m, WAVE);
    return r;
  }
};

// combines across the aligned groups of WIDTH lanes (a power of two, the whole wave by default); lane 0 of a
// group ends with its result.  The steps for a narrower group are the last steps of the wave's.
template <typename R, int WIDTH = WAVE>
__device__ __forceinline__ typename R::acc_t wave_reduce(typename R::acc_t a) {
#pragma unroll
  for (int m = WIDTH / 2; m >= 1; m >>= 1) a = R::combine(a, R::shfl_xor(a, m));
  return a;
}

template <typename CT>
__device__ __forceinline__ void finalize(void *out, int odt, int64_t o, CT v) { store_one<CT>(out, odt, o, v); }
template <typename CT>
__device__ __forceinline__ void finalize(void *out, int odt, int64_t o, ArgAcc<CT> a) {
  store_one<int64_t>(out, odt, o, (int64_t)a.i);
}

}  // namespace hipnx
