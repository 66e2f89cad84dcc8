/* Unary elementwise operations y = f(x) for every element type.
 *
 * Semantics follow solid/include/solid/core/generic/unary_ops.h:203-672 with
 * the CPU function table (solid/include/solid/core/cpu/unary_ops_cpu.h:24-140)
 * and the type table of solid/src/core/cpu/template_unary.c:35-260:
 *   integers .. transcendental functions go through double and are cast back
 *               (:230-261); sqrt/log of non-positive signed values give 0
 *   floats .... one library call in the work type; negative is -1*x,
 *               reciprocal is 1/x (:284-334)
 *   complex ... explicit real formulas (:346-672); sqrt is ACM algorithm 312
 * Operations built from IEEE basic operations are bit-exact against the CPU;
 * transcendental functions differ from the host libm in the last bits.
 */
#pragma once
#include "och_dtypes.h"
#include "och_math.h"
#include <math.h>

namespace och {

/* ---- math wrappers selecting the float or double routine ----------------- */
#define OCH_MATH1(NAME, FN, DN) \
   template <class W> OCH_D W NAME(W x) { if constexpr (std::is_same<W, float>::value) return FN(x); else return DN(x); }
OCH_MATH1(m_sin, sinf, sin)       OCH_MATH1(m_cos, cosf, cos)       OCH_MATH1(m_tan, tanf, tan)
OCH_MATH1(m_sinh, och_sinhf, och_sinh) OCH_MATH1(m_cosh, och_coshf, och_cosh) OCH_MATH1(m_tanh, tanhf, och_tanh)   /* och_*: och_math.h */
OCH_MATH1(m_asin, asinf, asin)    OCH_MATH1(m_acos, acosf, acos)    OCH_MATH1(m_atan, atanf, atan)
OCH_MATH1(m_asinh, och_asinhf, och_asinh) OCH_MATH1(m_acosh, och_acoshf, och_acosh) OCH_MATH1(m_atanh, och_atanhf, och_atanh)
OCH_MATH1(m_sqrt, sqrtf, sqrt)    OCH_MATH1(m_cbrt, cbrtf, cbrt)
OCH_MATH1(m_exp, expf, exp)       OCH_MATH1(m_exp2, exp2f, exp2)    OCH_MATH1(m_expm1, expm1f, expm1)
OCH_MATH1(m_log, logf, log)       OCH_MATH1(m_log2, log2f, log2)    OCH_MATH1(m_log10, log10f, log10)
OCH_MATH1(m_log1p, och_log1pf, och_log1p)
OCH_MATH1(m_fabs, fabsf, fabs)    OCH_MATH1(m_ceil, ceilf, ceil)    OCH_MATH1(m_floor, floorf, floor)
OCH_MATH1(m_trunc, truncf, trunc) OCH_MATH1(m_round, roundf, round)
#undef OCH_MATH1
/* sine and cosine of one argument share their argument reduction */
template <class W> OCH_D void m_sincos(W x, W &s, W &c) { if constexpr (std::is_same<W, float>::value) sincosf(x, &s, &c); else sincos(x, &s, &c); }
template <class W> OCH_D W m_atan2(W y, W x) { if constexpr (std::is_same<W, float>::value) return atan2f(y, x); else return atan2(y, x); }
template <class W> OCH_D W m_hypot(W x, W y) { if constexpr (std::is_same<W, float>::value) return hypotf(x, y); else return hypot(x, y); }
template <class W> OCH_D W m_copysign(W x, W y) { if constexpr (std::is_same<W, float>::value) return copysignf(x, y); else return copysign(x, y); }
/* pow in the CPU table: powf for BOTH float and double (och_math.h: the correctly rounded power in all but one case in 10^5) */
template <class W> OCH_D W m_pow(W x, W y) { return (W)och_powf((float)x, (float)y); }
/* exp10(x) is evaluated as exp(ln10 * x) */
template <class W> OCH_D W m_exp10(W x)
{  if constexpr (std::is_same<W, float>::value) return expf(((float)2.3025850929940459) * x);
   else return exp(2.3025850929940459 * x);
}
template <class W> OCH_D W c_ln2()  { return (W)0.69314718055994529; }
template <class W> OCH_D W c_ln10() { return (W)2.3025850929940459; }
template <class W> OCH_D W c_inf()  { return (W)(__builtin_huge_val()); }

enum UnaryId {
   U_NEGATIVE, U_BITWISE_NOT, U_LOGICAL_NOT, U_CONJ, U_RECIPROCAL,
   U_SIN, U_COS, U_TAN, U_SINH, U_COSH, U_TANH,
   U_ARCSIN, U_ARCCOS, U_ARCTAN, U_ARCSINH, U_ARCCOSH, U_ARCTANH,
   U_SQRT, U_CBRT, U_SQUARE, U_EXP, U_EXP2, U_EXP10, U_EXPM1,
   U_LOG, U_LOG2, U_LOG10, U_LOG1P,
   U_ABSOLUTE, U_FABS, U_SIGN, U_CEIL, U_FLOOR, U_TRUNC, U_ROUND,
   U_ISINF, U_ISNAN, U_ISFINITE, U_ISPOSINF, U_ISNEGINF, U_COUNT
};

/* real library function by id, in work type W */
template <int ID, class W> OCH_D W real_fun(W x)
{
   if constexpr (ID == U_SIN) return m_sin(x);          else if constexpr (ID == U_COS) return m_cos(x);
   else if constexpr (ID == U_TAN) return m_tan(x);     else if constexpr (ID == U_SINH) return m_sinh(x);
   else if constexpr (ID == U_COSH) return m_cosh(x);   else if constexpr (ID == U_TANH) return m_tanh(x);
   else if constexpr (ID == U_ARCSIN) return m_asin(x); else if constexpr (ID == U_ARCCOS) return m_acos(x);
   else if constexpr (ID == U_ARCTAN) return m_atan(x); else if constexpr (ID == U_ARCSINH) return m_asinh(x);
   else if constexpr (ID == U_ARCCOSH) return m_acosh(x); else if constexpr (ID == U_ARCTANH) return m_atanh(x);
   else if constexpr (ID == U_SQRT) return m_sqrt(x);   else if constexpr (ID == U_CBRT) return m_cbrt(x);
   else if constexpr (ID == U_EXP) return m_exp(x);     else if constexpr (ID == U_EXP2) return m_exp2(x);
   else if constexpr (ID == U_EXP10) return m_exp10(x); else if constexpr (ID == U_EXPM1) return m_expm1(x);
   else if constexpr (ID == U_LOG) return m_log(x);     else if constexpr (ID == U_LOG2) return m_log2(x);
   else if constexpr (ID == U_LOG10) return m_log10(x); else if constexpr (ID == U_LOG1P) return m_log1p(x);
   else if constexpr (ID == U_CEIL) return m_ceil(x);   else if constexpr (ID == U_FLOOR) return m_floor(x);
   else if constexpr (ID == U_TRUNC) return m_trunc(x); else if constexpr (ID == U_ROUND) return m_round(x);
   else if constexpr (ID == U_FABS) return m_fabs(x);
   else return x;
}

/* result type: bool for the is* queries, the part type for complex absolute, else T */
template <class T, int ID> struct unary_result
{  typedef typename std::conditional<(ID >= U_ISINF), obool,
           typename std::conditional<(ID == U_ABSOLUTE && is_complex_v<T>), typename traits<T>::elem, T>::type>::type type;
};

/* which (operation, type) pairs exist (the reference's LUT holds 0 elsewhere) */
template <class T, int ID> constexpr bool unary_defined()
{
   if (ID == U_NEGATIVE)    return !is_uint_v<T>;
   if (ID == U_BITWISE_NOT) return is_int_v<T> || is_bool_v<T>;
   if (ID == U_LOGICAL_NOT) return is_bool_v<T>;
   if (ID == U_CONJ)        return is_complex_v<T>;
   if (ID >= U_RECIPROCAL && ID <= U_LOG1P) return !is_bool_v<T>;
   if (ID >= U_CEIL && ID <= U_ROUND) return is_float_v<T> || is_complex_v<T>;
   if (ID == U_ISPOSINF || ID == U_ISNEGINF) return !is_complex_v<T>;
   return true;
}

template <class T, int ID> struct UnaryOp
{
   typedef T A;
   typedef typename unary_result<T, ID>::type R;

   static OCH_D R f(A x)
   {
      /* ---------------- queries ---------------- */
      if constexpr (ID >= U_ISINF)
      {  R y;
         if constexpr (is_bool_v<T> || is_int_v<T>) y.v = (ID == U_ISFINITE) ? 1 : 0;
         else if constexpr (is_float_v<T>)
         {  typename traits<T>::work w = to_work(x);
            if constexpr (ID == U_ISINF) y.v = isinf(w) ? 1 : 0;
            else if constexpr (ID == U_ISNAN) y.v = isnan(w) ? 1 : 0;
            else if constexpr (ID == U_ISFINITE) y.v = isfinite(w) ? 1 : 0;
            else if constexpr (ID == U_ISPOSINF) y.v = ((w > 0) && isinf(w)) ? 1 : 0;
            else y.v = ((w < 0) && isinf(w)) ? 1 : 0;
         }
         else
         {  elemwork_t<T> re = to_work(x.real), im = to_work(x.imag);
            if constexpr (ID == U_ISINF) y.v = (isinf(re) || isinf(im)) ? 1 : 0;
            else if constexpr (ID == U_ISNAN) y.v = (isnan(re) || isinf(im)) ? 1 : 0;   /* sic: the imaginary part is tested with isinf */
            else y.v = (isfinite(re) && isfinite(im)) ? 1 : 0;
         }
         return y;
      }
      /* ---------------- bool ---------------- */
      else if constexpr (is_bool_v<T>)
      {  R y;
         if constexpr (ID == U_NEGATIVE || ID == U_BITWISE_NOT || ID == U_LOGICAL_NOT) y.v = x.v ^ 1;
         else y.v = x.v;                                   /* fabs, sign, absolute */
         return y;
      }
      /* ---------------- integers ---------------- */
      else if constexpr (is_int_v<T>)
      {
         if constexpr (ID == U_BITWISE_NOT) return (T)~x;
         else if constexpr (ID == U_NEGATIVE)
         {  typedef typename std::make_unsigned<T>::type U; return (T)((U)0 - (U)x); }
         else if constexpr (ID == U_RECIPROCAL)
         {  if (x == 0) return (T)0;
            if constexpr (is_sint_v<T>) return (T)((x == 1) ? 1 : (x == -1) ? -1 : 0);
            else return (T)((x == 1) ? 1 : 0);
         }
         else if constexpr (ID == U_SQUARE)
         {  typedef typename std::make_unsigned<T>::type U;
            if constexpr (sizeof(T) < 4) return (T)((uint32_t)(U)x * (uint32_t)(U)x);
            else return (T)((U)x * (U)x);
         }
         else if constexpr (ID == U_FABS || ID == U_ABSOLUTE)
         {  if constexpr (is_uint_v<T>) return x;
            else { typedef typename std::make_unsigned<T>::type U; return (x < 0) ? (T)((U)0 - (U)x) : x; }
         }
         else if constexpr (ID == U_SIGN)
         {  if constexpr (is_uint_v<T>) return (T)(x > 0);
            else return (T)((x > 0) - (x < 0));
         }
         else if constexpr (ID == U_SQRT || ID == U_LOG || ID == U_LOG2 || ID == U_LOG10)
         {  if constexpr (is_sint_v<T>) { if (x <= 0) return (T)0; }
            return float_to_int<T, double>(real_fun<ID, double>((double)x));
         }
         else if constexpr (ID == U_LOG1P)
         {  double d = (double)x;
            if constexpr (is_sint_v<T>) { if (d <= -1) return (T)0; }
            return float_to_int<T, double>(m_log1p(d));
         }
         else return float_to_int<T, double>(real_fun<ID, double>((double)x));
      }
      /* ---------------- real floating point ---------------- */
      else if constexpr (is_float_v<T>)
      {  typedef typename traits<T>::work W;
         W w = to_work(x);
         if constexpr (ID == U_NEGATIVE) return from_work<T>((W)-1 * w);
         else if constexpr (ID == U_RECIPROCAL) return from_work<T>((W)1 / w);
         else if constexpr (ID == U_SQUARE) return from_work<T>(w * w);
         else if constexpr (ID == U_SIGN) { if (isnan(w)) return x; return from_work<T>((W)((w > 0) - (w < 0))); }
         else if constexpr (ID == U_ABSOLUTE) return from_work<T>(m_fabs(w));
         else return from_work<T>(real_fun<ID, W>(w));
      }
      /* ---------------- complex ---------------- */
      else
      {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W;
         W xr = to_work(x.real), xi = to_work(x.imag);
         if constexpr (ID == U_ABSOLUTE) return from_work<E>(m_hypot(xr, xi));
         else
         {  R y; W yr, yi;
            const E ezero = cvt_real<E>((uint8_t)0);
            if constexpr (ID == U_NEGATIVE) { yr = (W)-1 * xr; yi = (W)-1 * xi; }
            else if constexpr (ID == U_CONJ) { y.real = x.real; y.imag = from_work<E>((W)-1 * xi); return y; }
            else if constexpr (ID == U_RECIPROCAL)
            {  W scale = (W)1 / ((xr * xr) + (xi * xi)); yr = xr * scale; yi = xi * scale * (W)-1; }
            else if constexpr (ID == U_SIN)  { W sn, cs; m_sincos(xr, sn, cs); yr = sn * m_cosh(xi);  yi = cs * m_sinh(xi); }
            else if constexpr (ID == U_COS)  { W sn, cs; m_sincos(xr, sn, cs); yr = cs * m_cosh(xi);  yi = sn * m_sinh(xi) * (W)-1; }
            else if constexpr (ID == U_TAN)
            {  W a = 2 * xr, b = 2 * xi, sn, cs; m_sincos(a, sn, cs); W r = cs + m_cosh(b); yr = sn / r; yi = m_sinh(b) / r; }
            else if constexpr (ID == U_SINH) { W sn, cs; m_sincos(xi, sn, cs); yr = m_sinh(xr) * cs;  yi = m_cosh(xr) * sn; }
            else if constexpr (ID == U_COSH) { W sn, cs; m_sincos(xi, sn, cs); yr = m_cosh(xr) * cs;  yi = m_sinh(xr) * sn; }
            else if constexpr (ID == U_TANH)
            {  W a = 2 * xr, b = 2 * xi, sn, cs; m_sincos(b, sn, cs); W r = (W)1 / (m_cosh(a) + cs); yr = m_sinh(a) * r; yi = sn * r; }
            else if constexpr (ID == U_ARCSIN || ID == U_ARCCOS)
            {  W v1 = 1 - (xr * xr) + (xi * xi), v2 = -2 * xr * xi;
               W gamma = m_sqrt(m_hypot(v1, v2)), theta = m_atan2(v2, v1) / 2, sn, cs;
               m_sincos(theta, sn, cs);
               if constexpr (ID == U_ARCSIN) { v1 = -xi + gamma * cs; v2 = xr + gamma * sn; }
               else                          { v1 = xr - gamma * sn; v2 = xi + gamma * cs; }
               yr = m_atan2(v2, v1); yi = m_log(v1 * v1 + v2 * v2) / -2;
            }
            else if constexpr (ID == U_ARCTAN)
            {  W v1 = xr * xr, v2 = xi * xi;
               yr = m_atan2(2 * xr, 1 - v1 - v2) / 2;
               v2 = 1 + xi;
               yi = m_log(1 - 4 * xi / (v2 * v2 + v1)) / -4;
            }
            else if constexpr (ID == U_ARCSINH || ID == U_ARCCOSH)
            {  W v1, v2;
               if constexpr (ID == U_ARCSINH) v1 = 1 + (xr * xr) - (xi * xi); else v1 = (xr * xr) - (xi * xi) - 1;
               v2 = 2 * xr * xi;
               W gamma = m_sqrt(m_hypot(v1, v2)), theta = m_atan2(v2, v1) / 2, sn, cs;
               m_sincos(theta, sn, cs);
               v1 = xr + gamma * cs; v2 = xi + gamma * sn;
               yr = m_log(v1 * v1 + v2 * v2) / 2; yi = m_atan2(v2, v1);
            }
            else if constexpr (ID == U_ARCTANH)
            {  /* arctanh(z) = log((1+z)/(1-z)) / 2. The reference stores both terms into the
                  imaginary part, so its real part is never written (unary_ops.h:472-474);
                  this kernel stores the logarithm term as the real part. */
               W v1 = xr * xr, v2 = xi * xi;
               yi = m_atan2(2 * xi, 1 - v1 - v2) / 2;
               v1 = 1 - xr;
               yr = m_log(1 + 4 * xr / (v1 * v1 + v2)) / 4;
            }
            else if constexpr (ID == U_SQRT)
            {  W v = m_hypot(xr, xi);
               if (!(v > 0)) { y.real = from_work<E>(v); y.imag = y.real; return y; }
               else if (isinf(xi))
               {  /* the half-precision infinity constant of the CPU table is 0xFC00 */
                  if constexpr (std::is_same<E, half_t>::value) y.real.v = 0xFC00; else y.real = c_inf<W>();
                  y.imag = x.imag; return y;
               }
               else if (isinf(xr)) { yr = (xr > 0) ? xr : 0; yi = m_copysign((xr < 0) ? xr : (W)0, xi); }
               else if (xr >= 0) { v = m_sqrt((xr + v) * (W)0.5); yr = v; yi = xi / (2 * v); }
               else { v = m_sqrt((-xr + v) * (W)0.5); yr = ((xi >= 0) ? xi : -xi) / (2 * v); yi = m_copysign(v, xi); }
            }
            else if constexpr (ID == U_CBRT)
            {  W scale = (xr * xr) + (xi * xi);
               if (scale > 0)
               {  scale = m_pow(scale, (W)(1. / 6)); W angle = m_atan2(xi, xr) / 3, sn, cs;
                  m_sincos(angle, sn, cs);
                  yr = scale * cs; yi = scale * sn;
               }
               else { y.real = ezero; y.imag = ezero; return y; }
            }
            else if constexpr (ID == U_SQUARE) { yr = xr * xr - xi * xi; yi = 2 * xr * xi; }
            else if constexpr (ID == U_EXP)   { W s = m_exp(xr), sn, cs; m_sincos(xi, sn, cs); yr = s * cs; yi = s * sn; }
            else if constexpr (ID == U_EXP2)  { W b = xi * c_ln2<W>();  W s = m_exp2(xr), sn, cs;  m_sincos(b, sn, cs); yr = s * cs; yi = s * sn; }
            else if constexpr (ID == U_EXP10) { W b = xi * c_ln10<W>(); W s = m_exp10(xr), sn, cs; m_sincos(b, sn, cs); yr = s * cs; yi = s * sn; }
            else if constexpr (ID == U_EXPM1) { W s = m_exp(xr), sn, cs; m_sincos(xi, sn, cs); yr = s * cs - 1; yi = s * sn; }
            else if constexpr (ID == U_LOG)   { W s = xr * xr + xi * xi; yr = m_log(s) * (W)0.5;   yi = m_atan2(xi, xr); }
            else if constexpr (ID == U_LOG2)  { W s = xr * xr + xi * xi; yr = m_log2(s) * (W)0.5;  yi = m_atan2(xi, xr) / c_ln2<W>(); }
            else if constexpr (ID == U_LOG10) { W s = xr * xr + xi * xi; yr = m_log10(s) * (W)0.5; yi = m_atan2(xi, xr) / c_ln10<W>(); }
            else if constexpr (ID == U_LOG1P) { W a = xr + 1; W s = a * a + xi * xi; yr = m_log(s) * (W)0.5; yi = m_atan2(xi, a); }
            else if constexpr (ID == U_FABS)  { y.real = from_work<E>(m_hypot(xr, xi)); y.imag = ezero; return y; }
            else if constexpr (ID == U_SIGN)
            {  if (isnan(xr) || isnan(xi)) yr = xr + xi;
               else yr = (W)(((xr > 0) - (xr < 0)) + (xr == 0) * ((xi > 0) - (xi < 0)));
               y.real = from_work<E>(yr); y.imag = ezero; return y;
            }
            else if constexpr (ID == U_CEIL)  { yr = m_ceil(xr);  yi = m_ceil(xi); }
            else if constexpr (ID == U_FLOOR) { yr = m_floor(xr); yi = m_floor(xi); }
            else if constexpr (ID == U_TRUNC) { yr = m_trunc(xr); yi = m_trunc(xi); }
            else if constexpr (ID == U_ROUND) { yr = m_round(xr); yi = m_round(xi); }
            else { yr = xr; yi = xi; }
            y.real = from_work<E>(yr); y.imag = from_work<E>(yi);
            return y;
         }
      }
   }
};

/* fill_nan: replace NaN entries by a value (unary_ops.h:332-334,669-672) */
template <class T> OCH_D bool fillnan_test(T x)
{
   if constexpr (is_float_v<T>) return isnan(to_work(x));
   else if constexpr (is_complex_v<T>) return isnan(to_work(x.real)) || isinf(to_work(x.imag));  /* sic */
   else return false;
}

} /* namespace och */
