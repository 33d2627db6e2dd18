// Correctly rounded float64 quotients without the division sequence.  Plain C++ with compiler
// built-ins only: the kernels include it with MIST_ARITH_FN = `__device__ __forceinline__`, the
// CPU test that pins these identities against IEEE division builds it with a host compiler.
#pragma once

#ifndef MIST_ARITH_FN
#define MIST_ARITH_FN static inline
#endif

namespace mist_arith {

// Bounds of the quotient inside which quotient_by_reciprocal() is exact (see there).
constexpr double kQuotientTiny = 0x1p-800;
constexpr double kQuotientHuge = 0x1p800;
// Divisors the fast path is used with: callers check them on the host.
constexpr double kDivisorMin = 0x1p-100;
constexpr double kDivisorMax = 0x1p100;

// True when quotient_by_reciprocal(a, b, 1 / b) may be used for a / b; `q0` = a * (1 / b).
// Zero dividends are exact trivially; infinities, NaNs and quotients near the ends of the
// exponent range go to the ordinary division.
MIST_ARITH_FN bool quotient_is_tame(double a, double q0) {
  const double mag = __builtin_fabs(q0);
  return (mag > kQuotientTiny && mag < kQuotientHuge) || a == 0.0;
}

// a / b, correctly rounded, from y = RN(1 / b) (itself from one real division, shared by many
// quotients with the same divisor): q0 = RN(a y) is within 1.5 ulp of a / b; one residual step
// (r = a - b q0 by FMA, q1 = RN(q0 + r y)) leaves a faithful q1, and for a faithful q1 and a
// correctly rounded y the second residual step returns RN(a / b) (Markstein's theorem; no
// underflow or overflow for kDivisorMin <= b <= kDivisorMax and the quotient range above, where
// both residuals are exact multiples of representable units).  Five multiply-add operations
// instead of the ~14 of the division sequence with its reciprocal at quarter rate.
// kKeepNegativeZero = false saves the final select for callers whose dividend is never -0.
template <bool kKeepNegativeZero = true>
MIST_ARITH_FN double quotient_by_reciprocal(double a, double b, double y, double q0) {
  double r = __builtin_fma(-b, q0, a);
  double q = __builtin_fma(r, y, q0);
  r = __builtin_fma(-b, q, a);
  q = __builtin_fma(r, y, q);
  if (!kKeepNegativeZero) return q;
  return a == 0.0 ? q0 : q;  // the residual steps would turn -0 into +0
}

// numpy's float64 floor_divide(a, b) for finite a >= 0, b > 0 with a / b < 2^50: the exact
// integer floor(a / b).  (npy_divmod takes mod = fmod(a, b), div = (a - mod) / b and rounds div
// to the nearest integer below or at it, with a half-way correction: for these operands
// (a - mod) / b is the exact integer quotient up to two roundings, which that correction
// absorbs.)  Here: the rounded quotient's floor, moved by one where the exact residual
// a - n b (one FMA: its sign and its comparison with b survive the rounding) says so.
MIST_ARITH_FN bool floor_divide_is_tame(double a, double b) {
  return a >= 0.0 && b >= kDivisorMin && b <= kDivisorMax && a < 0x1p50 * b && a < kQuotientHuge;
}

MIST_ARITH_FN double floor_divide_tame(double a, double b) {
  double n = __builtin_floor(a / b);
  const double r = __builtin_fma(-n, b, a);
  if (r < 0.0) n -= 1.0;
  else if (r >= b) n += 1.0;
  return n;
}

}  // namespace mist_arith
