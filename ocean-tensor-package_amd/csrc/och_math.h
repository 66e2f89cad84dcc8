/* Two elementary functions written out in IEEE basic operations: powf and tanh (double).
 *
 * The device math library's routines for these two cost more arithmetic than the memory system leaves time for (powf
 * about 210 instructions per element, tanh on double about 140 double-precision operations, most of them the
 * double-double arithmetic of its extended exponential); a streaming kernel built on them runs at half the rate of its
 * neighbours. The routines below need a third of that. They use additions, multiplications, fused multiply-adds,
 * divisions, conversions and integer operations on the bits only -- no library call -- so a host build of this header
 * gives bit for bit what the device gives, and the accuracy against the host's libm (the reference's CPU functions:
 * solid/include/solid/core/cpu/unary_ops_cpu.h:24-140, powf for the power of both float and double) is established on the
 * CPU over millions of arguments and every special case.
 *
 *   och_powf(x, y)   |x|^y as exp2(y * log2|x|) in double precision: log2 from the exponent and an atanh series of
 *                    (m - 1) / (m + 1) for the mantissa m in [0.707, 1.414), exp2 from the nearest integer and a
 *                    degree-9 polynomial. The double result is some thousand times more accurate than a float's last
 *                    place, so its rounding to float is the correctly rounded power except where the true value lies
 *                    within 1e-11 of the middle between two floats (the host's powf is off by one unit in the last
 *                    place a hundred times as often). Signs, zeros, infinities and NaNs follow C99 F.10.4.4, as the
 *                    host's powf does.
 *   och_tanh(x)      E / (E + 2) with E = exp(2|x|) - 1 built without cancellation from a reduction by ln 2 in two parts
 *                    and a degree-13 polynomial for e^g - 1; 1 from 20 on. Within 2 units in the last place of the
 *                    host's tanh.
 */
#pragma once
#include <stdint.h>

#ifndef OCH_MATH_FN
#  if defined(__HIPCC__)
#     define OCH_MATH_FN __host__ __device__ __forceinline__
#  else
#     define OCH_MATH_FN static inline
#  endif
#endif

namespace och {

OCH_MATH_FN double   math_from_bits(uint64_t u) { union { uint64_t u; double d; } c; c.u = u; return c.d; }
OCH_MATH_FN uint64_t math_to_bits(double d)     { union { uint64_t u; double d; } c; c.d = d; return c.u; }
OCH_MATH_FN float    math_float_from_bits(uint32_t u) { union { uint32_t u; float f; } c; c.u = u; return c.f; }
OCH_MATH_FN uint32_t math_float_to_bits(float f)      { union { uint32_t u; float f; } c; c.f = f; return c.u; }

/* 2^k for -1022 <= k <= 1023 */
OCH_MATH_FN double math_pow2i(int k) { return math_from_bits((uint64_t)(k + 1023) << 52); }

/* a^y for a positive, finite, normal double a and a finite y, both converted from floats; the result to be rounded to
   float. Relative error below 1e-11 (a float's last place is 6e-8):
     log2 a = e + log2 m, m in [0.707, 1.414): log m = 2 atanh s = 2 s (1 + z / 3 + ... + z^7 / 15), s = (m - 1) / (m + 1),
              z = s^2 <= 0.0295 (truncation 3e-14 of log m; the error of log2 a counts |y log2 a| ln 2 <= 104 times)
     2^p    = 2^k e^((p - k) ln 2), k the nearest integer: Taylor polynomial of degree 9 (truncation 7e-12) */
OCH_MATH_FN double math_pow_core(double a, double y)
{
   const uint64_t u = math_to_bits(a);
   int e = (int)(u >> 52) - 1023;
   double m = math_from_bits((u & 0x000FFFFFFFFFFFFFull) | 0x3FF0000000000000ull);       /* [1, 2) */
   const bool upper = m >= 1.4142135623730951;
   m = upper ? m * 0.5 : m;
   e = upper ? e + 1 : e;
   const double s = (m - 1.0) / (m + 1.0), z = s * s;
   double t = 1.0 / 15.0;
   t = __builtin_fma(t, z, 1.0 / 13.0); t = __builtin_fma(t, z, 1.0 / 11.0); t = __builtin_fma(t, z, 1.0 / 9.0);
   t = __builtin_fma(t, z, 1.0 / 7.0);  t = __builtin_fma(t, z, 1.0 / 5.0);  t = __builtin_fma(t, z, 1.0 / 3.0);
   const double two_s = s + s;
   const double logm = __builtin_fma(two_s * z, t, two_s);
   double p = y * __builtin_fma(logm, 1.4426950408889634074 /* 1 / ln 2 */, (double)e);
   p = p > 200.0 ? 200.0 : p;                                    /* 2^200 and 2^-200 are infinity and zero as floats */
   p = p < -200.0 ? -200.0 : p;
   const double k = __builtin_rint(p);
   const double g = (p - k) * 0.69314718055994530942;
   double q = 1.0 / 362880.0;
   q = __builtin_fma(q, g, 1.0 / 40320.0); q = __builtin_fma(q, g, 1.0 / 5040.0); q = __builtin_fma(q, g, 1.0 / 720.0);
   q = __builtin_fma(q, g, 1.0 / 120.0);   q = __builtin_fma(q, g, 1.0 / 24.0);   q = __builtin_fma(q, g, 1.0 / 6.0);
   q = __builtin_fma(q, g, 0.5);           q = __builtin_fma(q, g, 1.0);          q = __builtin_fma(q, g, 1.0);
   return q * math_pow2i((int)k);
}

/* the arguments of the plain case: 0 < x < inf and y finite (x = 1 and y = 0 give 1 by themselves there) */
OCH_MATH_FN bool math_powf_plain(float x, float y)
{  return math_float_to_bits(x) - 1u < 0x7F7FFFFFu && (math_float_to_bits(y) & 0x7FFFFFFFu) < 0x7F800000u; }

/* every case, C99 F.10.4.4 */
OCH_MATH_FN float math_powf_any(float x, float y)
{
   const uint32_t bx = math_float_to_bits(x), by = math_float_to_bits(y);
   const uint32_t ax = bx & 0x7FFFFFFFu, ay = by & 0x7FFFFFFFu;
   const bool xneg = (bx >> 31) != 0, yneg = (by >> 31) != 0;
   /* is y an integer, and an odd one? From 2^24 on every float is an even integer (so is an infinity, for the rules below) */
   const float fay = math_float_from_bits(ay);
   const bool ybig = ay >= 0x4B800000u;
   const int iy = ybig ? 0 : (int)fay;
   const bool yint = ybig || (float)iy == fay;
   const bool yodd = !ybig && yint && (iy & 1);
   /* the general case on sanitised arguments: |x| finite and positive, |y| finite */
   const bool xfinite = ax - 1u < 0x7F7FFFFFu;                   /* 0 < |x| < inf */
   const bool yfinite = ay < 0x7F800000u;
   float mag = (float)math_pow_core(xfinite ? (double)math_float_from_bits(ax) : 1.0, yfinite ? (double)y : 0.0);
   const float inf = math_float_from_bits(0x7F800000u), nan = math_float_from_bits(0x7FC00000u);
   if (ax == 0x7F800000u) mag = yneg ? 0.0f : inf;                                            /* |x| = inf */
   if (ax == 0) mag = yneg ? inf : 0.0f;                                                      /* x = +-0 */
   if (!yfinite) mag = (ax == 0x3F800000u) ? 1.0f : (((ax > 0x3F800000u) != yneg) ? inf : 0.0f);      /* y = +-inf */
   float z = (xneg && yodd) ? -mag : mag;
   if (xneg && !yint && xfinite) z = nan;                                                     /* negative base, fractional exponent */
   if (ax > 0x7F800000u || ay > 0x7F800000u) z = nan;                                         /* a NaN argument ... */
   if (ay == 0 || bx == 0x3F800000u) z = 1.0f;                                                /* ... unless y = 0 or x = 1 */
   return z;
}

OCH_MATH_FN float och_powf(float x, float y)
{
#if defined(__HIP_DEVICE_COMPILE__)
   /* positive finite bases with finite exponents take the plain case without a divergent branch; a wave with any other
      argument pair runs the complete routine for those lanes (the empty asm statement keeps the compiler from
      evaluating it unconditionally) */
   const bool plain = math_powf_plain(x, y);
   float z = (float)math_pow_core(plain ? (double)x : 1.0, plain ? (double)y : 0.0);
   if (__builtin_amdgcn_ballot_w64(!plain) != 0)
   {  asm volatile("" ::: "memory");
      if (!plain) z = math_powf_any(x, y);
   }
   return z;
#else
   return math_powf_plain(x, y) ? (float)math_pow_core((double)x, (double)y) : math_powf_any(x, y);
#endif
}

OCH_MATH_FN double och_tanh(double x)
{
   const uint64_t bx = math_to_bits(x);
   const double a = math_from_bits(bx & 0x7FFFFFFFFFFFFFFFull);
   /* tanh a = E / (E + 2) with E = e^2a - 1 = 2^k (e^g - 1) + (2^k - 1), 2a = k ln 2 + g: no difference of nearly equal
      numbers anywhere, so small arguments need no series of their own (k = 0: E = e^g - 1 = g + g^2 / 2 + ...). From 20 on
      the quotient is 1 to the last place; the clamp keeps k small and NaN out of the integer conversion. */
   const double u = a < 20.0 ? a + a : 40.0;
   const double k = __builtin_rint(u * 1.4426950408889634074);
   double g = __builtin_fma(k, -6.93147180369123816490e-01, u);          /* ln 2 in two parts: the first has 32 bits ... */
   g = __builtin_fma(k, -1.90821492927058770002e-10, g);                   /* ... so its products with k are exact */
   double q = 1.0 / 6227020800.0;                                          /* (e^g - 1 - g) / g^2 = 1/2 + g/6 + ... + g^11 / 13! */
   q = __builtin_fma(q, g, 1.0 / 479001600.0); q = __builtin_fma(q, g, 1.0 / 39916800.0); q = __builtin_fma(q, g, 1.0 / 3628800.0);
   q = __builtin_fma(q, g, 1.0 / 362880.0);    q = __builtin_fma(q, g, 1.0 / 40320.0);    q = __builtin_fma(q, g, 1.0 / 5040.0);
   q = __builtin_fma(q, g, 1.0 / 720.0);       q = __builtin_fma(q, g, 1.0 / 120.0);      q = __builtin_fma(q, g, 1.0 / 24.0);
   q = __builtin_fma(q, g, 1.0 / 6.0);         q = __builtin_fma(q, g, 0.5);
   const double em1 = __builtin_fma(g * g, q, g);
   const double pk = math_pow2i((int)k);
   const double E = __builtin_fma(pk, em1, pk - 1.0);
   /* E / (E + 2) with the rounding of the sum taken back: D + lost = E + 2 exactly (E < 2: the larger term is 2) */
   const double D = E + 2.0;
   const double lost = E < 2.0 ? E - (D - 2.0) : 2.0 - (D - E);
   const double rcp = 1.0 / D;
   const double r0 = E * rcp;
   double r = __builtin_fma(__builtin_fma(-r0, lost, __builtin_fma(-r0, D, E)), rcp, r0);
   r = math_from_bits(math_to_bits(r) | (bx & 0x8000000000000000ull));
   return a == a ? r : x + x;                                               /* NaN stays NaN */
}

} /* namespace och */
