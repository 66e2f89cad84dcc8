/* Elementary functions written out in IEEE basic operations: powf, tanh (double), sinh, cosh, log1p, asinh, acosh, atanh.
 *
 * The device math library's routines for these cost more arithmetic than the memory system leaves time for (powf about
 * 210 instructions per element, tanh on double about 140 double-precision operations, most of them the double-double
 * arithmetic of its extended exponential; sinh, cosh, log1p and the inverse hyperbolic functions 125 to 200 instructions
 * in either precision, against the 48 (float) and 96 (double) that fit under the memory time of a unary kernel); a
 * streaming kernel built on them runs at half the rate of its neighbours or less. The routines below need a third to a
 * half of that. The float versions evaluate in double precision with shorter polynomials and round once. They use additions, multiplications, fused multiply-adds,
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
 *   och_sinh, och_cosh   from the same exponential: (E + E / (E + 1)) / 2 below 1, e^a / 2 -+ 1 / (2 e^a) above, overflowing
 *                    where the functions do (not where e^a does). Within 3 units in the last place of the host's.
 *   och_log1p, och_atanh, och_asinh, och_acosh   fdlibm's formulas (s_log1p.c, e_atanh.c, s_asinh.c, e_acosh.c) on a log of
 *                    this file's own (atanh series of (m - 1) / (m + 1), e ln 2 added in two parts), every case of each
 *                    function as one log1p of a selected argument. Within 3 units in the last place of the host's.
 *   och_*f           the same in double precision with shorter series, rounded to float once: within 2 units of the
 *                    host's float functions (which are themselves not correctly rounded).
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

/* ---- hyperbolic sine and cosine ----------------------------------------------------------------------------------
   e^u for u >= 0 in two parts: k, the nearest integer to u / ln 2, and e^g - 1 for the rest g (|g| <= 0.347), which is
   g + g^2 (1/2 + g/6 + ...) without a rounded 1 in it. FULL: degree 13, for results in double; otherwise degree 9
   (relative truncation 2e-11), for results that are rounded to float. */
template <bool FULL>
OCH_MATH_FN double math_exp_rest(double u, double &k)
{
   k = __builtin_rint(u * 1.4426950408889634074);
   double g = __builtin_fma(k, -6.93147180369123816490e-01, u);
   g = __builtin_fma(k, -1.90821492927058770002e-10, g);
   double q;
   if (FULL)
   {  q = 1.0 / 6227020800.0;
      q = __builtin_fma(q, g, 1.0 / 479001600.0); q = __builtin_fma(q, g, 1.0 / 39916800.0); q = __builtin_fma(q, g, 1.0 / 3628800.0);
      q = __builtin_fma(q, g, 1.0 / 362880.0);
   }
   else q = 1.0 / 362880.0;
   q = __builtin_fma(q, g, 1.0 / 40320.0); q = __builtin_fma(q, g, 1.0 / 5040.0); q = __builtin_fma(q, g, 1.0 / 720.0);
   q = __builtin_fma(q, g, 1.0 / 120.0);   q = __builtin_fma(q, g, 1.0 / 24.0);   q = __builtin_fma(q, g, 1.0 / 6.0);
   q = __builtin_fma(q, g, 0.5);
   return __builtin_fma(g * g, q, g);
}

/* e^a / 2 for 0 <= a <= 711 without an early overflow: (e^g 2^(k - 1 - c)) 2^c, c = 64 for the largest k */
OCH_MATH_FN double math_half_exp(double em1, double k)
{
   const int ik = (int)k, c = ik > 1000 ? 64 : 0;
   return ((em1 + 1.0) * math_pow2i(ik - 1 - c)) * math_pow2i(c);
}

/* sinh a = (E + E / (E + 1)) / 2 with E = e^a - 1 below 1 (no cancellation: E = 2^k (e^g - 1) + (2^k - 1), k = 0 or 1),
   e^a / 2 - 1 / (2 e^a) from 1 on; cosh a = e^a / 2 + 1 / (2 e^a). Overflow to infinity where the functions overflow
   (710.4758...), not where e^a does. */
template <bool FULL>
OCH_MATH_FN double math_sinh(double x)
{
   const uint64_t bx = math_to_bits(x);
   const double a = math_from_bits(bx & 0x7FFFFFFFFFFFFFFFull);
   double k;
   const double em1 = math_exp_rest<FULL>(a < 711.0 ? a : 711.0, k);
   const double pk = k < 2.0 ? k + 1.0 : 1.0;                              /* 2^k for k = 0, 1 (only used below 1) */
   const double E = __builtin_fma(pk, em1, pk - 1.0);
   const double th = math_half_exp(em1, k);
   const bool small = a < 1.0;
   const double q = (small ? E : 0.25) / (small ? E + 1.0 : th);          /* one division for both forms */
   double r = small ? 0.5 * (E + q) : th - q;
   r = math_from_bits(math_to_bits(r) | (bx & 0x8000000000000000ull));
   return a == a ? r : x + x;
}
template <bool FULL>
OCH_MATH_FN double math_cosh(double x)
{
   const double a = math_from_bits(math_to_bits(x) & 0x7FFFFFFFFFFFFFFFull);
   double k;
   const double em1 = math_exp_rest<FULL>(a < 711.0 ? a : 711.0, k);
   const double th = math_half_exp(em1, k);
   const double r = th + 0.25 / th;
   return a == a ? r : x + x;
}
OCH_MATH_FN double och_sinh(double x) { return math_sinh<true>(x); }
OCH_MATH_FN double och_cosh(double x) { return math_cosh<true>(x); }
OCH_MATH_FN float  och_sinhf(float x) { return (float)math_sinh<false>((double)x); }
OCH_MATH_FN float  och_coshf(float x) { return (float)math_cosh<false>((double)x); }

/* ---- log1p and the inverse hyperbolic functions ---------------------------------------------------------------------
   log of a positive normal double: v = 2^e m with m in [0.707, 1.414), f = m - 1, log m = 2 atanh s = 2 s + s R with
   s = f / (2 + f), z = s^2 <= 0.0295, R = z (2/3 + 2/5 z + 2/7 z^2 + ...). FULL: terms up to 2/19 z^9 (truncation 2e-17);
   otherwise up to 2/11 z^5 (1e-10, for results rounded to float). math_log_parts returns e, f and the small part of
   log m = f - tail; e ln 2 is added in two parts. */
template <bool FULL>
OCH_MATH_FN void math_log_parts(double v, double &de, double &f, double &tail)
{
   const uint64_t u = math_to_bits(v);
   int e = (int)(u >> 52) - 1023;
   double m = math_from_bits((u & 0x000FFFFFFFFFFFFFull) | 0x3FF0000000000000ull);
   const bool upper = m >= 1.4142135623730951;
   m = upper ? m * 0.5 : m;
   e = upper ? e + 1 : e;
   f = m - 1.0;                                                             /* exact */
   const double s = f / (2.0 + f), z = s * s;
   double t;
   if (FULL)
   {  t = 2.0 / 19.0;
      t = __builtin_fma(t, z, 2.0 / 17.0); t = __builtin_fma(t, z, 2.0 / 15.0); t = __builtin_fma(t, z, 2.0 / 13.0);
      t = __builtin_fma(t, z, 2.0 / 11.0);
   }
   else t = 2.0 / 11.0;
   t = __builtin_fma(t, z, 2.0 / 9.0); t = __builtin_fma(t, z, 2.0 / 7.0); t = __builtin_fma(t, z, 2.0 / 5.0);
   t = __builtin_fma(t, z, 2.0 / 3.0);
   /* log m = 2 s + s R, R = z t; with 2 s = f - s f and f^2 / 2 split off: log m = f - (f^2 / 2 - s (f^2 / 2 + R)), the
      arrangement of fdlibm's e_log.c: the leading term is exact and everything after it is small */
   const double hfsq = 0.5 * f * f;
   tail = hfsq - s * __builtin_fma(z, t, hfsq);                             /* log m = f - tail */
   de = (double)e;
}
template <bool FULL>
OCH_MATH_FN double math_log_normal(double v)
{
   double de, f, tail;
   math_log_parts<FULL>(v, de, f, tail);
   return __builtin_fma(de, 6.93147180369123816490e-01, -((tail - de * 1.90821492927058770002e-10) - f));
}

/* log(1 + y) for y > -1, finite: the log of the rounded sum plus what the rounding took away, (y - (u - 1)) / u */
template <bool FULL>
OCH_MATH_FN double math_log1p_core(double y)
{
   const double u = 1.0 + y;
   /* for a result rounded to float the lost part matters only where u is within 2^-29 of 1: no division by u there */
   const double c = FULL ? ((u - 1.0 == y) ? 0.0 : (y - (u - 1.0)) / u) : y - (u - 1.0);
   return math_log_normal<FULL>(u) + c;
}

template <bool FULL>
OCH_MATH_FN double math_log1p(double x)
{
   const double inf = math_from_bits(0x7FF0000000000000ull);
   const bool plain = x > -1.0 && x < inf;
   double r = math_log1p_core<FULL>(plain ? x : 0.0);
   /* 1 + x = 1 for tiny x: the correction term alone gives x (also for -0 and subnormal x, where log 1 + x / 1 = x) */
   if (x == 0.0) r = x;                                                    /* keeps the sign of zero */
   if (x == inf) r = inf;
   if (x == -1.0) r = -inf;
   if (x < -1.0 || x != x) r = math_from_bits(0x7FF8000000000000ull);
   return r;
}

/* atanh a = log1p(2a / (1 - a)) / 2, below 0.5 as log1p(2a + 2a a / (1 - a)) / 2 (e_atanh.c of fdlibm) */
template <bool FULL>
OCH_MATH_FN double math_atanh(double x)
{
   const uint64_t bx = math_to_bits(x);
   const double a = math_from_bits(bx & 0x7FFFFFFFFFFFFFFFull);
   const bool plain = a < 1.0;
   const double b = plain ? a : 0.0, t = b + b, q = b / (1.0 - b);                  /* (2a / (1 - a) = 2 q: one division) */
   double r = 0.5 * math_log1p_core<FULL>(b < 0.5 ? __builtin_fma(t, q, t) : q + q);
   if (a == 1.0) r = math_from_bits(0x7FF0000000000000ull);
   r = math_from_bits(math_to_bits(r) | (bx & 0x8000000000000000ull));
   if (a > 1.0 || a != a) r = math_from_bits(0x7FF8000000000000ull);
   return r;
}

/* asinh a = log1p(a + a^2 / (1 + sqrt(1 + a^2))) up to 2, log(a + sqrt(a^2 + 1)) = log1p((a - 1) + sqrt(a^2 + 1)) above (no
   cancellation there), log a + log 2 from 2^28 on (the cases of s_asinh.c of fdlibm); all three as one log1p */
template <bool FULL>
OCH_MATH_FN double math_asinh(double x)
{
   const uint64_t bx = math_to_bits(x);
   const double a = math_from_bits(bx & 0x7FFFFFFFFFFFFFFFull);
   const bool big = a >= 268435456.0, finite = a < math_from_bits(0x7FF0000000000000ull);
   const double b = (big || !finite) ? 1.0 : a, t = b * b, root = __builtin_sqrt(t + 1.0);
   const double low = b + t / (1.0 + root);
   const double high = (b - 1.0) + root;
   double w = b <= 2.0 ? low : high;
   w = big && finite ? a - 1.0 : w;
   double r = math_log1p_core<FULL>(w) + (big ? 6.93147180559945286227e-01 : 0.0);
   r = finite ? r : a;                                                      /* infinity, NaN */
   r = math_from_bits(math_to_bits(r) | (bx & 0x8000000000000000ull));
   return a == a ? r : x + x;
}

/* acosh x = log(x + sqrt(x^2 - 1)) = log1p(t + sqrt(t^2 + 2 t)), t = x - 1: sums of positive terms for every x >= 1;
   log x + log 2 from 2^28 on (e_acosh.c of fdlibm has the same cases with a log instead of a log1p above 2) */
template <bool FULL>
OCH_MATH_FN double math_acosh(double x)
{
   const double inf = math_from_bits(0x7FF0000000000000ull);
   const bool big = x >= 268435456.0, plain = x >= 1.0 && x < inf;
   const double b = (plain && !big) ? x : 1.0, t = b - 1.0;
   double w = t + __builtin_sqrt(__builtin_fma(t, t, t + t));
   w = big && plain ? x - 1.0 : w;
   double r = math_log1p_core<FULL>(w) + ((big && plain) ? 6.93147180559945286227e-01 : 0.0);
   if (x == inf) r = inf;
   if (x < 1.0 || x != x) r = math_from_bits(0x7FF8000000000000ull);
   return r;
}

OCH_MATH_FN double och_log1p(double x) { return math_log1p<true>(x); }
OCH_MATH_FN double och_atanh(double x) { return math_atanh<true>(x); }
OCH_MATH_FN double och_asinh(double x) { return math_asinh<true>(x); }
OCH_MATH_FN double och_acosh(double x) { return math_acosh<true>(x); }
OCH_MATH_FN float  och_log1pf(float x) { return (float)math_log1p<false>((double)x); }
OCH_MATH_FN float  och_atanhf(float x) { return (float)math_atanh<false>((double)x); }
OCH_MATH_FN float  och_asinhf(float x) { return (float)math_asinh<false>((double)x); }
OCH_MATH_FN float  och_acoshf(float x) { return (float)math_acosh<false>((double)x); }

} /* namespace och */
