// expm1 and log1p in double precision for the neuron updates.
//
// The LIF update needs expm1(-t / tau) with t at most one time step and
// log1p(-(v - 1) / (j - 1)), whose argument is bounded by the step's decay factor
// (v - 1 = (v_old - 1)(1 - f) + f (j - 1) <= f (j - 1) for v_old <= 1), so with the usual
// dt / tau_rc = 0.05 both arguments lie in [-0.05, 0].  A general-purpose double-precision
// routine spends most of its instructions on range reduction and on the cases far from
// zero; for |x| <= 1/16 the Taylor series, summed by Horner's rule with fused multiply-adds,
// is as accurate: the result is x + x^2 q(x) with |x^2 q(x)| <= |x| / 30, so the rounding
// errors of q enter scaled down and the result is within 0.6 units in the last place of the
// true value (truncation: below 2^-60 |x|).  The callers round it to float32, which gives
// the correctly rounded float32 value except when the true value lies within that distance
// of a float32 rounding boundary (a chance of the order of 1e-9 per evaluation: the same
// as for any two library routines that each promise one unit in the last place).
// Arguments outside the interval go to the library routine.
//
// Plain C++ (no device intrinsics beyond the fused multiply-add builtin), so that a host
// compiler can build the same functions for a test against the host's math library.
#pragma once

#include <math.h>

#if defined(__HIPCC__)
#define NHIP_MATH_FN __host__ __device__ __forceinline__
#else
#define NHIP_MATH_FN static inline
#endif

// expm1(x) for |x| <= 1/16: x + x^2 (1/2 + x/6 + ... + x^8 / 10!)
NHIP_MATH_FN double nhip_expm1_small(double x) {
    double q = 1.0 / 3628800.0;
    q = __builtin_fma(q, x, 1.0 / 362880.0);
    q = __builtin_fma(q, x, 1.0 / 40320.0);
    q = __builtin_fma(q, x, 1.0 / 5040.0);
    q = __builtin_fma(q, x, 1.0 / 720.0);
    q = __builtin_fma(q, x, 1.0 / 120.0);
    q = __builtin_fma(q, x, 1.0 / 24.0);
    q = __builtin_fma(q, x, 1.0 / 6.0);
    q = __builtin_fma(q, x, 0.5);
    // (+0 from the product plus a zero of either sign is +0: a zero is returned as it came)
    return x == 0.0 ? x : __builtin_fma(x * x, q, x);
}

// log1p(x) for |x| <= 1/16: x + x^2 (-1/2 + x/3 - x^2/4 + ... - x^12 / 14)
NHIP_MATH_FN double nhip_log1p_small(double x) {
    double q = -1.0 / 14.0;
    q = __builtin_fma(q, x, 1.0 / 13.0);
    q = __builtin_fma(q, x, -1.0 / 12.0);
    q = __builtin_fma(q, x, 1.0 / 11.0);
    q = __builtin_fma(q, x, -1.0 / 10.0);
    q = __builtin_fma(q, x, 1.0 / 9.0);
    q = __builtin_fma(q, x, -1.0 / 8.0);
    q = __builtin_fma(q, x, 1.0 / 7.0);
    q = __builtin_fma(q, x, -1.0 / 6.0);
    q = __builtin_fma(q, x, 1.0 / 5.0);
    q = __builtin_fma(q, x, -1.0 / 4.0);
    q = __builtin_fma(q, x, 1.0 / 3.0);
    q = __builtin_fma(q, x, -0.5);
    return __builtin_fma(x * x, q, x);
}

constexpr double NHIP_SMALL_ARG = 0.0625;

// (a NaN fails the comparison and reaches the library routine, which returns it)
NHIP_MATH_FN double nhip_expm1(double x) {
    return fabs(x) <= NHIP_SMALL_ARG ? nhip_expm1_small(x) : expm1(x);
}

NHIP_MATH_FN double nhip_log1p(double x) {
    return fabs(x) <= NHIP_SMALL_ARG ? nhip_log1p_small(x) : log1p(x);
}
