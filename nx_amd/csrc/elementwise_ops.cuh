// Scalar semantics of the element-wise callbacks, shared by the streaming kernels.
//
// Compute classes.  The reference decodes every element to an Erlang number (IEEE double or
// unbounded integer), applies the operation and encodes once (nx/lib/nx/binary_backend.ex:
// 662-706, 2432-2438).  The same value is obtained on the device with
//   float   when every operand is exactly representable in f32 and the output is f32/bf16/f16
//           (a correctly rounded f32 + - * / equals the f64 operation rounded to f32);
//   double  for every other combination that involves a float;
//   int64_t (two's-complement wrap) when operands and output are integers.
#pragma once
#ifndef __HIPCC_RTC__
#include <type_traits>
#include <utility>
#endif

#include "dtypes.cuh"

namespace hipnx {

template <typename T> struct is_fp { static constexpr bool value = false; };
template <> struct is_fp<float> { static constexpr bool value = true; };
template <> struct is_fp<double> { static constexpr bool value = true; };

constexpr bool binary_int_only(int op) {
  return op == HIPNX_QUOTIENT || (op >= HIPNX_BITWISE_AND && op <= HIPNX_RIGHT_SHIFT);
}
constexpr bool binary_float_only(int op) { return op == HIPNX_DIVIDE || op == HIPNX_ATAN2; }
// ops whose integer result depends on reading the operands as signed or unsigned 64-bit
constexpr bool binary_sign_matters(int op) {
  return op == HIPNX_REMAINDER || op == HIPNX_QUOTIENT || op == HIPNX_MIN || op == HIPNX_MAX ||
         op == HIPNX_RIGHT_SHIFT || (op >= HIPNX_GREATER && op <= HIPNX_LESS_EQUAL) || op == HIPNX_POW;
}

// Operand pairs the reference raises for instead of returning a value (binary_backend.ex:711-750):
// codes of the deferred error word (the top byte; the low 56 bits carry the offending operand).
enum {
  HIPNX_RAISE_NONE = 0,
  HIPNX_RAISE_BADARITH = 1,     // div/2, rem/2 by zero; :math.fmod/2 with a zero divisor
  HIPNX_RAISE_LEFT_SHIFT = 2,   // "cannot left shift by <n>"
  HIPNX_RAISE_RIGHT_SHIFT = 3,  // "cannot right shift by <n>"
  HIPNX_RAISE_NEG_EXPONENT = 4, // Integer.pow/2 with a negative exponent
  HIPNX_RAISE_NOT_A_NUMBER = 5, // :math.fmod/2 of a non-finite element
  HIPNX_RAISE_INDEX = 6         // gather index out of bounds (deferred policy)
};
constexpr bool binary_can_raise(int op, bool fp) {
  return fp ? op == HIPNX_REMAINDER
            : (op == HIPNX_QUOTIENT || op == HIPNX_REMAINDER || op == HIPNX_LEFT_SHIFT || op == HIPNX_RIGHT_SHIFT || op == HIPNX_POW);
}
template <int OP, typename CT, bool UNS>
__device__ __forceinline__ int binary_raises(CT a, CT b, long long *operand) {
  if constexpr (is_fp<CT>::value) {
    if constexpr (OP == HIPNX_REMAINDER) {
      if (a != a || b != b || a - a != 0 || b - b != 0) return HIPNX_RAISE_NOT_A_NUMBER;
      if (b == 0) return HIPNX_RAISE_BADARITH;
    }
  } else {
    *operand = (long long)b;
    if constexpr (OP == HIPNX_QUOTIENT || OP == HIPNX_REMAINDER) {
      if (b == 0) return HIPNX_RAISE_BADARITH;
    } else if constexpr (OP == HIPNX_LEFT_SHIFT) {
      if (!UNS && b < 0) return HIPNX_RAISE_LEFT_SHIFT;
    } else if constexpr (OP == HIPNX_RIGHT_SHIFT) {
      if (!UNS && b < 0) return HIPNX_RAISE_RIGHT_SHIFT;
    } else if constexpr (OP == HIPNX_POW) {
      if (!UNS && b < 0) return HIPNX_RAISE_NEG_EXPONENT;
    }
  }
  return HIPNX_RAISE_NONE;
}
// the report: one 8-byte store to the context's pinned host word (any of the offending lanes may win)
__device__ __forceinline__ void report_raise(unsigned long long *err, int code, long long operand) {
  __hip_atomic_store(err, ((unsigned long long)code << 56) | ((unsigned long long)operand & 0x00FFFFFFFFFFFFFFull),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ int64_t ipow_wrap(int64_t base, uint64_t e) {
  uint64_t r = 1, b = (uint64_t)base;
  while (e) {
    if (e & 1) r *= b;
    b *= b;
    e >>= 1;
  }
  return (int64_t)r;
}

// element_* of nx/lib/nx/binary_backend.ex:708-816
template <int OP, typename CT, bool UNS>
__device__ __forceinline__ CT binary_apply(CT a, CT b) {
  if constexpr (is_fp<CT>::value) {
    if constexpr (OP == HIPNX_ADD) return a + b;
    else if constexpr (OP == HIPNX_SUBTRACT) return a - b;
    else if constexpr (OP == HIPNX_MULTIPLY) return a * b;
    else if constexpr (OP == HIPNX_DIVIDE) return a / b;
    else if constexpr (OP == HIPNX_POW) return pow(a, b);
    else if constexpr (OP == HIPNX_REMAINDER) return fmod(a, b);
    else if constexpr (OP == HIPNX_ATAN2) {
      // through f64, as the reference computes it (one rounding of the f64 result).  The f32 routine of the device
      // library comes in two variants (one with a faster division), and the offline and the run-time compiler do not
      // pick the same one: a fused group compiled at run time would differ from the same node run alone in the last bit.
      return (CT)atan2((double)a, (double)b);
    }
    else if constexpr (OP == HIPNX_MAX) return (a != a || b != b) ? (CT)NAN : (b > a ? b : a);
    else if constexpr (OP == HIPNX_MIN) return (a != a || b != b) ? (CT)NAN : (b < a ? b : a);
    else if constexpr (OP == HIPNX_EQUAL) return (CT)(a == b);
    else if constexpr (OP == HIPNX_NOT_EQUAL) return (CT)(a != b);
    else if constexpr (OP == HIPNX_GREATER) return (CT)(a > b);
    else if constexpr (OP == HIPNX_LESS) return (CT)(a < b);
    else if constexpr (OP == HIPNX_GREATER_EQUAL) return (CT)(a >= b);
    else if constexpr (OP == HIPNX_LESS_EQUAL) return (CT)(a <= b);
    else if constexpr (OP == HIPNX_LOGICAL_AND) return (CT)((a != 0) && (b != 0));
    else if constexpr (OP == HIPNX_LOGICAL_OR) return (CT)((a != 0) || (b != 0));
    else if constexpr (OP == HIPNX_LOGICAL_XOR) return (CT)((a != 0) != (b != 0));
    else return (CT)0;  // integer-only ops never reach a float class
  } else {
    typedef typename std::conditional<UNS, uint64_t, int64_t>::type S;
    const uint64_t ua = (uint64_t)a, ub = (uint64_t)b;
    const S sa = (S)a, sb = (S)b;
    if constexpr (OP == HIPNX_ADD) return (int64_t)(ua + ub);
    else if constexpr (OP == HIPNX_SUBTRACT) return (int64_t)(ua - ub);
    else if constexpr (OP == HIPNX_MULTIPLY) return (int64_t)(ua * ub);
    else if constexpr (OP == HIPNX_POW) return (!UNS && b < 0) ? 0 : ipow_wrap(a, ub);
    else if constexpr (OP == HIPNX_REMAINDER) {
      if (sb == 0) return 0;  // the reference raises ArithmeticError
      if (!UNS && b == -1) return 0;
      return (int64_t)(sa % sb);
    } else if constexpr (OP == HIPNX_QUOTIENT) {
      if (sb == 0) return 0;  // the reference raises ArithmeticError
      if (!UNS && b == -1) return (int64_t)(0 - ua);
      return (int64_t)(sa / sb);
    } else if constexpr (OP == HIPNX_MAX) return sb > sa ? b : a;
    else if constexpr (OP == HIPNX_MIN) return sb < sa ? b : a;
    else if constexpr (OP == HIPNX_BITWISE_AND) return a & b;
    else if constexpr (OP == HIPNX_BITWISE_OR) return a | b;
    else if constexpr (OP == HIPNX_BITWISE_XOR) return a ^ b;
    else if constexpr (OP == HIPNX_LEFT_SHIFT) return ((!UNS && b < 0) || ub >= 64) ? 0 : (int64_t)(ua << b);
    else if constexpr (OP == HIPNX_RIGHT_SHIFT) {
      if (b < 0) return 0;  // the reference raises ArgumentError
      if (b >= 64) return (!UNS && a < 0) ? -1 : 0;
      return (int64_t)(sa >> b);
    } else if constexpr (OP == HIPNX_EQUAL) return a == b;
    else if constexpr (OP == HIPNX_NOT_EQUAL) return a != b;
    else if constexpr (OP == HIPNX_GREATER) return sa > sb;
    else if constexpr (OP == HIPNX_LESS) return sa < sb;
    else if constexpr (OP == HIPNX_GREATER_EQUAL) return sa >= sb;
    else if constexpr (OP == HIPNX_LESS_EQUAL) return sa <= sb;
    else if constexpr (OP == HIPNX_LOGICAL_AND) return (a != 0) && (b != 0);
    else if constexpr (OP == HIPNX_LOGICAL_OR) return (a != 0) || (b != 0);
    else if constexpr (OP == HIPNX_LOGICAL_XOR) return (a != 0) != (b != 0);
    else return 0;  // float-only ops never reach the integer class
  }
}

// erf_inv as the reference computes it (Complex.erf_inv of the `complex` package, called from
// nx/lib/nx/shared.ex:373-375): Giles' single-precision polynomial evaluated in f64 -- its error
// of a few 1e-7 relative is part of the reference result, so it is followed term by term
// (products and sums round separately; the unit is compiled without contraction).  The
// reference's known answers that pin it: nx/lib/nx/random.ex:514-533, nx/test/nx/random_test.exs:141-165.
__device__ __forceinline__ double erf_inv_reference(double x) {
  if (x != x || x < -1.0 || x > 1.0) return __builtin_nan("");
  if (x == 1.0) return __builtin_inf();
  if (x == -1.0) return -__builtin_inf();
  if (x == 0.0) return x;
  double w = -log((1.0 - x) * (1.0 + x)), p;
  if (w < 5.0) {
    w = w - 2.5;
    p = 2.81022636e-08;
    p = 3.43273939e-07 + p * w;
    p = -3.5233877e-06 + p * w;
    p = -4.39150654e-06 + p * w;
    p = 0.00021858087 + p * w;
    p = -0.00125372503 + p * w;
    p = -0.00417768164 + p * w;
    p = 0.246640727 + p * w;
    p = 1.50140941 + p * w;
  } else {
    w = sqrt(w) - 3.0;
    p = -0.000200214257;
    p = 0.000100950558 + p * w;
    p = 0.00134934322 + p * w;
    p = -0.00367342844 + p * w;
    p = 0.00573950773 + p * w;
    p = -0.0076224613 + p * w;
    p = 0.00943887047 + p * w;
    p = 1.00167406 + p * w;
    p = 2.83297682 + p * w;
  }
  return p * x;
}

constexpr bool unary_int_only(int op) {
  return op == HIPNX_BITWISE_NOT || op == HIPNX_CLZ || op == HIPNX_POPCOUNT;
}
constexpr bool unary_is_math(int op) { return op <= HIPNX_ERF_INV; }

// nx/lib/nx/shared.ex:311-376 (formulas, e.g. expm1 = exp(x) - 1 and log1p = log(x + 1) exactly
// as written there) and nx/lib/nx/binary_backend.ex:834-1003.  `bits` is the input width.
template <int OP, typename CT>
__device__ __forceinline__ CT unary_apply(CT x, int bits) {
  if constexpr (is_fp<CT>::value) {
    if constexpr (OP == HIPNX_EXP) return exp(x);
    // the cancellation in these three is part of the reference result: follow it in f64
    else if constexpr (OP == HIPNX_EXPM1) return (CT)(exp((double)x) - 1.0);
    else if constexpr (OP == HIPNX_LOG1P) return (CT)log((double)x + 1.0);
    else if constexpr (OP == HIPNX_SIGMOID) return (CT)(1.0 / (exp(-(double)x) + 1.0));
    else if constexpr (OP == HIPNX_LOG) return log(x);
    else if constexpr (OP == HIPNX_COS) return cos(x);
    else if constexpr (OP == HIPNX_SIN) return sin(x);
    else if constexpr (OP == HIPNX_TAN) return tan(x);
    else if constexpr (OP == HIPNX_COSH) return cosh(x);
    else if constexpr (OP == HIPNX_SINH) return sinh(x);
    else if constexpr (OP == HIPNX_TANH) return tanh(x);
    else if constexpr (OP == HIPNX_ACOS) return acos(x);
    else if constexpr (OP == HIPNX_ASIN) return asin(x);
    else if constexpr (OP == HIPNX_ATAN) return atan(x);
    else if constexpr (OP == HIPNX_ACOSH) return acosh(x);
    else if constexpr (OP == HIPNX_ASINH) return asinh(x);
    else if constexpr (OP == HIPNX_ATANH) return atanh(x);
    else if constexpr (OP == HIPNX_SQRT) return sqrt(x);
    else if constexpr (OP == HIPNX_RSQRT) return (CT)1 / sqrt(x);
    else if constexpr (OP == HIPNX_CBRT) return cbrt(x);
    else if constexpr (OP == HIPNX_ERF) return erf(x);
    else if constexpr (OP == HIPNX_ERFC) return erfc(x);
    else if constexpr (OP == HIPNX_ERF_INV) return (CT)erf_inv_reference((double)x);
    else if constexpr (OP == HIPNX_ABS) return fabs(x);
    else if constexpr (OP == HIPNX_CEIL) return ceil(x);
    else if constexpr (OP == HIPNX_FLOOR) return floor(x);
    else if constexpr (OP == HIPNX_NEGATE) return -x;
    else if constexpr (OP == HIPNX_ROUND) return round(x);  // half away from zero
    else if constexpr (OP == HIPNX_SIGN) {
      // guards `n < 0` / `n > 0` run in Erlang term order, where the atoms :nan, :infinity and
      // :neg_infinity all sort above every number: each of them yields 1
      if (x != x || isinf(x)) return (CT)1;
      return x < 0 ? (CT)-1 : (x > 0 ? (CT)1 : x);
    } else if constexpr (OP == HIPNX_IS_NAN) return (CT)(x != x);
    else if constexpr (OP == HIPNX_IS_INFINITY) return (CT)(isinf(x) ? 1 : 0);
    else return (CT)0;
  } else {
    uint64_t u = (uint64_t)x;
    if (bits < 64) u &= (1ull << bits) - 1;
    if constexpr (OP == HIPNX_ABS) return x < 0 ? (int64_t)(0 - (uint64_t)x) : x;
    else if constexpr (OP == HIPNX_NEGATE) return (int64_t)(0 - (uint64_t)x);
    else if constexpr (OP == HIPNX_BITWISE_NOT) return ~x;
    else if constexpr (OP == HIPNX_SIGN) return x < 0 ? -1 : (x > 0 ? 1 : 0);
    else if constexpr (OP == HIPNX_CLZ) return u == 0 ? bits : (int64_t)(__clzll((long long)u) - (64 - bits));
    else if constexpr (OP == HIPNX_POPCOUNT) return (int64_t)__popcll(u);
    else if constexpr (OP == HIPNX_CEIL || OP == HIPNX_FLOOR || OP == HIPNX_ROUND) return x;
    else return 0;  // is_nan / is_infinity of an integer
  }
}

// as_type float -> integer (nx/lib/nx/binary_backend.ex:2049-2069): trunc toward zero as an
// unbounded integer whose low bits are kept; NaN -> 0, +Inf -> max, -Inf -> min of the type.
__device__ __forceinline__ int64_t float_to_int_wrap(double d, int64_t tmax, int64_t tmin) {
  if (d != d) return 0;
  if (isinf(d)) return d > 0 ? tmax : tmin;
  double t = trunc(d);
  if (fabs(t) < 9.2e18) return (int64_t)t;
  double m = fmod(t, 18446744073709551616.0);  // exact, in (-2^64, 2^64)
  if (m < 0) m += 18446744073709551616.0;     // exact: both are multiples of the same ulp
  uint64_t u = m >= 9223372036854775808.0 ? ((uint64_t)(m - 9223372036854775808.0) | (1ull << 63)) : (uint64_t)m;
  return (int64_t)u;
}

}  // namespace hipnx
