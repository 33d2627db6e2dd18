// Host build of mist_amd/csrc/exact_arith.h for tests/test_exact_arith.py: the same source the
// kernels compile, called on arrays.
#include "exact_arith.h"

extern "C" {

// out[i] = a[i] / b[i] through the reciprocal path; tame[i] = 0 where the kernels would take the
// division sequence instead (out[i] is then left untouched).
void quotients_by_reciprocal(const double *a, const double *b, double *out, unsigned char *tame,
                             long n) {
  for (long i = 0; i < n; ++i) {
    const bool divisor_ok = b[i] >= mist_arith::kDivisorMin && b[i] <= mist_arith::kDivisorMax;
    const double y = 1.0 / b[i];
    const double q0 = a[i] * y;
    tame[i] = divisor_ok && mist_arith::quotient_is_tame(a[i], q0);
    if (tame[i]) out[i] = mist_arith::quotient_by_reciprocal(a[i], b[i], y, q0);
  }
}

// The same for dividends that are never -0 (the variant without the final select).
void quotients_by_reciprocal_no_negative_zero(const double *a, const double *b, double *out,
                                              unsigned char *tame, long n) {
  for (long i = 0; i < n; ++i) {
    const bool divisor_ok = b[i] >= mist_arith::kDivisorMin && b[i] <= mist_arith::kDivisorMax;
    const double y = 1.0 / b[i];
    const double q0 = a[i] * y;
    tame[i] = divisor_ok && mist_arith::quotient_is_tame(a[i], q0);
    if (tame[i]) out[i] = mist_arith::quotient_by_reciprocal<false>(a[i], b[i], y, q0);
  }
}

void floor_divides(const double *a, const double *b, double *out, unsigned char *tame, long n) {
  for (long i = 0; i < n; ++i) {
    tame[i] = mist_arith::floor_divide_is_tame(a[i], b[i]);
    if (tame[i]) out[i] = mist_arith::floor_divide_tame(a[i], b[i]);
  }
}

}  // extern "C"
