/* Reduction operations: per (operation, element type) the accumulator type, the map from
 * an element to its contribution, the associative combine step and the final conversion.
 *
 * Semantics follow solid/include/solid/core/generic/reduce_ops.h:139-1287 (result types,
 * NaN rules, integer widening). Differences that are deliberate:
 *   - floating-point sums, products and norms accumulate in double (complex: a pair of
 *     doubles) and are combined as a tree; the CPU path folds serially in the input
 *     precision per thread, so its rounding depends on the thread count. Results agree to
 *     the documented tolerance and are closer to the exact value.
 *   - maximum / minimum start from a NaN accumulator instead of the first element; with the
 *     reference's update rule ("replace when the candidate is not NaN and the accumulator is
 *     not >= it") a NaN accumulator is displaced by the first number, so the result is the
 *     same: NaNs are ignored unless every element is NaN.
 *   - the NaN-skipping complex product uses the correct complex multiplication (the
 *     reference's accumulate step has a sign slip, reduce_ops.h:784).
 */
#pragma once
#include "och_dtypes.h"
#include "och_ops_unary.h"

namespace och {

enum ReduceId {
   R_ANY, R_ALL, R_ALL_FINITE, R_ANY_INF, R_ANY_NAN, R_NNZ, R_NNZ_NAN,
   R_ALL_LT, R_ALL_LE, R_ALL_GT, R_ALL_GE, R_ALL_GTLT, R_ALL_GTLE, R_ALL_GELT, R_ALL_GELE,
   R_SUM, R_SUM_NAN, R_PROD, R_PROD_NAN, R_SUM_ABS, R_SUM_ABS_NAN,
   R_MAXIMUM, R_MINIMUM, R_MAXIMUM_ABS, R_MINIMUM_ABS, R_NORM, R_NORM_NAN, R_NORM2, R_NORM2_NAN, R_COUNT
};

template <int OP> constexpr bool red_is_logical() { return OP <= R_ANY_NAN || (OP >= R_ALL_LT && OP <= R_ALL_GELE); }
/* all_finite / any_inf / any_nan exist for floating types only; the other *_nan variants
   are defined for every type and equal the plain operation on integers (the CPU functions
   forward, solid/src/core/cpu/template_reduce_all.c:373-376) */
template <int OP> constexpr bool red_is_float_only()
{  return OP == R_ALL_FINITE || OP == R_ANY_INF || OP == R_ANY_NAN; }

template <class T, int OP> constexpr bool reduce_defined()
{  return red_is_float_only<OP>() ? (is_float_v<T> || is_complex_v<T>) : true; }

struct dpair { double real, imag; };

/* work type of a complex element as a struct of two W */
template <class T> struct cwork { elemwork_t<T> real, imag; };

template <class T> struct red_param
{  T bound1, bound2;          /* in the tensor's own type */
   double phalf, pinv;        /* p/2 and 1/p for the general norm */
};

/* Complex maximum / minimum keep the FIRST element when every element has a NaN part (reduce_ops.h:912-935: the
   accumulator starts as the first element and only NaN-free elements replace it). A parallel reduction starts every
   partial from an identity, so the identity must lose against any element, NaN parts included: it is a quiet NaN with
   a payload that no arithmetic produces, recognised by its bits. */
template <class F> OCH_D F extreme_identity()
{  if constexpr (sizeof(F) == 4) { union { uint32_t u; float f; } c; c.u = 0x7FC0D1CEu; return c.f; }
   else { union { uint64_t u; double f; } c; c.u = 0x7FF8D1CED1CED1CEull; return c.f; }
}
template <class F> OCH_D bool is_extreme_identity(F v)
{  if constexpr (sizeof(F) == 4) { union { uint32_t u; float f; } c; c.f = v; return c.u == 0x7FC0D1CEu; }
   else { union { uint64_t u; double f; } c; c.f = v; return c.u == 0x7FF8D1CED1CED1CEull; }
}

/* pow of the general p-norm as one out-of-line function per translation unit: inlined at every load site of every
   kernel variant it multiplies the code size and the build time of the norm kernels */
static __device__ __noinline__ double norm_pow(double x, double y) { return pow(x, y); }

template <class T, int OP> struct Reduce
{
   typedef typename traits<T>::work W;
   typedef typename traits<T>::elem E;
   typedef typename traits<T>::abs  ABS;
   static constexpr bool LOGICAL = red_is_logical<OP>();
   static constexpr bool SUMLIKE = (OP == R_SUM || OP == R_SUM_NAN || OP == R_PROD || OP == R_PROD_NAN);
   static constexpr bool ABSSUM  = (OP == R_SUM_ABS || OP == R_SUM_ABS_NAN);
   static constexpr bool EXTREME = (OP == R_MAXIMUM || OP == R_MINIMUM);
   static constexpr bool ABSEXT  = (OP == R_MAXIMUM_ABS || OP == R_MINIMUM_ABS);
   static constexpr bool NORM    = (OP >= R_NORM);
   static constexpr bool ISMAX   = (OP == R_MAXIMUM || OP == R_MAXIMUM_ABS);
   static constexpr bool NEEDS_DATA = EXTREME || ABSEXT;     /* undefined for empty tensors */

   /* ---- accumulator ---- */
   typedef typename std::conditional<LOGICAL, uint32_t,
           typename std::conditional<(OP == R_NNZ || OP == R_NNZ_NAN), uint64_t,
           typename std::conditional<SUMLIKE,
              typename std::conditional<(is_bool_v<T> || is_uint_v<T>), uint64_t,
              typename std::conditional<is_sint_v<T>, int64_t,
              typename std::conditional<is_float_v<T>, double, dpair>::type>::type>::type,
           typename std::conditional<ABSSUM,
              typename std::conditional<(is_float_v<T> || is_complex_v<T>), double, uint64_t>::type,
           typename std::conditional<EXTREME,
              typename std::conditional<is_bool_v<T>, uint8_t,
              typename std::conditional<is_complex_v<T>, cwork<T>, W>::type>::type,
           typename std::conditional<ABSEXT,
              typename std::conditional<is_bool_v<T>, uint8_t,
              typename std::conditional<is_int_v<T>, ABS,
              typename std::conditional<is_complex_v<T>, elemwork_t<T>, W>::type>::type>::type,
           double>::type>::type>::type>::type>::type>::type Acc;

   /* ---- result storage type ---- */
   typedef typename std::conditional<LOGICAL, obool,
           typename std::conditional<(OP == R_NNZ || OP == R_NNZ_NAN), uint64_t,
           typename std::conditional<SUMLIKE,
              typename std::conditional<(is_bool_v<T> || is_uint_v<T>), uint64_t,
              typename std::conditional<is_sint_v<T>, int64_t, T>::type>::type,
           typename std::conditional<ABSSUM,
              typename std::conditional<(is_float_v<T> || is_complex_v<T>), ABS, uint64_t>::type,
           typename std::conditional<EXTREME, T,
           typename std::conditional<ABSEXT, ABS,
              typename std::conditional<(is_float_v<T> || is_complex_v<T>), ABS, double>::type>::type>::type>::type>::type>::type>::type Res;

   typedef red_param<T> Param;

   /* ---- identity ---- */
   static OCH_D Acc identity()
   {
      if constexpr (LOGICAL) return (OP == R_ANY || OP == R_ANY_INF || OP == R_ANY_NAN) ? 0u : 1u;
      else if constexpr (OP == R_NNZ || OP == R_NNZ_NAN) return 0;
      else if constexpr (SUMLIKE)
      {  constexpr bool P = (OP == R_PROD || OP == R_PROD_NAN);
         if constexpr (is_complex_v<T>) { dpair a; a.real = P ? 1.0 : 0.0; a.imag = 0.0; return a; }
         else return (Acc)(P ? 1 : 0);
      }
      else if constexpr (ABSSUM || NORM) return (Acc)0;
      else if constexpr (EXTREME)
      {  if constexpr (is_bool_v<T>) return ISMAX ? 0 : 1;
         else if constexpr (is_uint_v<T>) return ISMAX ? (T)0 : (T)~(T)0;
         else if constexpr (is_sint_v<T>)
         {  typedef typename std::make_unsigned<T>::type U;
            return ISMAX ? (T)((U)1 << (sizeof(T) * 8 - 1)) : (T)(((U)1 << (sizeof(T) * 8 - 1)) - 1);
         }
         else if constexpr (is_float_v<T>) return (W)__builtin_nan("");
         else { cwork<T> a; a.real = extreme_identity<elemwork_t<T>>(); a.imag = a.real; return a; }
      }
      else   /* ABSEXT */
      {  if constexpr (is_bool_v<T>) return ISMAX ? 0 : 1;
         else if constexpr (is_int_v<T>) return ISMAX ? (ABS)0 : (ABS)~(ABS)0;
         else return (Acc)__builtin_nan("");
      }
   }

   /* comparison against the bounds of the range checks */
   static OCH_D bool in_range(T x, const Param &p)
   {
      if constexpr (is_complex_v<T>)
      {  typedef elemwork_t<T> V;
         V re = to_work(x.real), im = to_work(x.imag);
         V lr = to_work(p.bound1.real), li = to_work(p.bound1.imag), ur = to_work(p.bound2.real), ui = to_work(p.bound2.imag);
         if constexpr (OP == R_ALL_LT) return !((re > lr) || ((re == lr) && (im >= li)));
         else if constexpr (OP == R_ALL_LE) return !((re > lr) || ((re == lr) && (im > li)));
         else if constexpr (OP == R_ALL_GT) return !((re < lr) || ((re == lr) && (im <= li)));
         else if constexpr (OP == R_ALL_GE) return !((re < lr) || ((re == lr) && (im < li)));
         else if constexpr (OP == R_ALL_GTLT) return !((re < lr) || (re > ur) || ((re == lr) && (im <= li)) || ((re == ur) && (im >= ui)));
         else if constexpr (OP == R_ALL_GTLE) return !((re < lr) || (re > ur) || ((re == lr) && (im <= li)) || ((re == ur) && (im >  ui)));
         else if constexpr (OP == R_ALL_GELT) return !((re < lr) || (re > ur) || ((re == lr) && (im <  li)) || ((re == ur) && (im >= ui)));
         else return !((re < lr) || (re > ur) || ((re == lr) && (im < li)) || ((re == ur) && (im > ui)));
      }
      else
      {  auto v = raw(x), lo = raw(p.bound1), hi = raw(p.bound2);
         if constexpr (OP == R_ALL_LT) return !(v >= lo);
         else if constexpr (OP == R_ALL_LE) return !(v > lo);
         else if constexpr (OP == R_ALL_GT) return !(v <= lo);
         else if constexpr (OP == R_ALL_GE) return !(v < lo);
         else if constexpr (OP == R_ALL_GTLT) return !((v <= lo) || (v >= hi));
         else if constexpr (OP == R_ALL_GTLE) return !((v <= lo) || (v >  hi));
         else if constexpr (OP == R_ALL_GELT) return !((v <  lo) || (v >= hi));
         else return !((v < lo) || (v > hi));
      }
   }

   /* real value in the work type (bool: its byte) */
   template <class X> static OCH_D auto raw(X x)
   {  if constexpr (is_bool_v<X>) return x.v; else return to_work(x); }

   /* ---- element -> contribution ---- */
   static OCH_D Acc load(T x, const Param &p)
   {
      if constexpr (OP == R_ANY || OP == R_NNZ)
      {  if constexpr (is_complex_v<T>) return (!(to_work(x.real) == 0) || !(to_work(x.imag) == 0)) ? 1 : 0;
         else return (!(raw(x) == 0)) ? 1 : 0;
      }
      else if constexpr (OP == R_ALL)
      {  if constexpr (is_complex_v<T>) return ((to_work(x.real) == 0) && (to_work(x.imag) == 0)) ? 0 : 1;
         else return (raw(x) == 0) ? 0 : 1;
      }
      else if constexpr (OP == R_ALL_FINITE)
      {  if constexpr (is_complex_v<T>) return (isfinite(to_work(x.real)) && isfinite(to_work(x.imag))) ? 1 : 0;
         else return isfinite(to_work(x)) ? 1 : 0;
      }
      else if constexpr (OP == R_ANY_INF)
      {  if constexpr (is_complex_v<T>) return (isinf(to_work(x.real)) || isinf(to_work(x.imag))) ? 1 : 0;
         else return isinf(to_work(x)) ? 1 : 0;
      }
      else if constexpr (OP == R_ANY_NAN)
      {  if constexpr (is_complex_v<T>) return (isnan(to_work(x.real)) || isnan(to_work(x.imag))) ? 1 : 0;
         else return isnan(to_work(x)) ? 1 : 0;
      }
      else if constexpr (OP == R_NNZ_NAN && !is_float_v<T> && !is_complex_v<T>) return (!(raw(x) == 0)) ? 1 : 0;
      else if constexpr (OP == R_NNZ_NAN)
      {  if constexpr (is_complex_v<T>)
         {  auto re = to_work(x.real), im = to_work(x.imag);
            return (!isnan(re) && !isnan(im) && ((re != 0) || (im != 0))) ? 1 : 0;
         }
         else { auto v = to_work(x); return (!isnan(v) && (v != 0)) ? 1 : 0; }
      }
      else if constexpr (LOGICAL) return in_range(x, p) ? 1u : 0u;
      else if constexpr (SUMLIKE)
      {  constexpr bool SKIP = (OP == R_SUM_NAN || OP == R_PROD_NAN);
         if constexpr (is_complex_v<T>)
         {  dpair a; a.real = (double)to_work(x.real); a.imag = (double)to_work(x.imag);
            if constexpr (SKIP) { if (isnan(a.real) || isnan(a.imag)) return identity(); }
            return a;
         }
         else if constexpr (is_float_v<T>)
         {  double v = (double)to_work(x);
            if constexpr (SKIP) { if (isnan(v)) return identity(); }
            return v;
         }
         else return (Acc)raw(x);
      }
      else if constexpr (ABSSUM)
      {  if constexpr (is_complex_v<T>)
         {  auto re = to_work(x.real), im = to_work(x.imag);
            if constexpr (OP == R_SUM_ABS_NAN) { if (isnan(re) || isnan(im)) return 0.0; }
            return (double)m_hypot(re, im);
         }
         else if constexpr (is_float_v<T>)
         {  auto v = to_work(x);
            if constexpr (OP == R_SUM_ABS_NAN) { if (isnan(v)) return 0.0; }
            return (double)m_fabs(v);
         }
         else if constexpr (is_sint_v<T>) return (x < 0) ? ((uint64_t)0 - (uint64_t)(int64_t)x) : (uint64_t)x;
         else return (uint64_t)raw(x);
      }
      else if constexpr (EXTREME)
      {  if constexpr (is_complex_v<T>) { cwork<T> a; a.real = to_work(x.real); a.imag = to_work(x.imag); return a; }
         else return raw(x);
      }
      else if constexpr (ABSEXT)
      {  if constexpr (is_complex_v<T>) return m_hypot(to_work(x.real), to_work(x.imag));
         else if constexpr (is_float_v<T>) return m_fabs(to_work(x));
         else if constexpr (is_sint_v<T>) return (x < 0) ? (ABS)((ABS)0 - (ABS)x) : (ABS)x;
         else return raw(x);
      }
      else   /* norms */
      {  double sq;
         if constexpr (is_complex_v<T>)
         {  double re = (double)to_work(x.real), im = (double)to_work(x.imag); sq = re * re + im * im; }
         else { double v = (double)raw(x); sq = v * v; }
         if constexpr (OP == R_NORM_NAN || OP == R_NORM2_NAN) { if (isnan(sq)) return 0.0; }
         if constexpr (OP == R_NORM || OP == R_NORM_NAN) return norm_pow(sq, p.phalf);
         else return sq;
      }
   }

   /* ---- associative combine ---- */
   static OCH_D Acc combine(Acc a, Acc b)
   {
      if constexpr (LOGICAL) return (OP == R_ANY || OP == R_ANY_INF || OP == R_ANY_NAN) ? (a | b) : (a & b);
      else if constexpr (OP == R_NNZ || OP == R_NNZ_NAN || ABSSUM || NORM) return a + b;
      else if constexpr (SUMLIKE)
      {  constexpr bool P = (OP == R_PROD || OP == R_PROD_NAN);
         if constexpr (is_complex_v<T>)
         {  dpair r;
            if constexpr (P) { r.real = a.real * b.real - a.imag * b.imag; r.imag = a.real * b.imag + a.imag * b.real; }
            else { r.real = a.real + b.real; r.imag = a.imag + b.imag; }
            return r;
         }
         else if constexpr (is_sint_v<T>)
         {  if constexpr (P) return (int64_t)((uint64_t)a * (uint64_t)b); else return (int64_t)((uint64_t)a + (uint64_t)b); }
         else { if constexpr (P) return a * b; else return a + b; }
      }
      else if constexpr (EXTREME && is_complex_v<T>)
      {  if (is_extreme_identity(a.real) && is_extreme_identity(a.imag)) return b;
         bool take = (!isnan(b.real)) && (!isnan(b.imag)) &&
                     (ISMAX ? ((!(a.real >= b.real)) || ((!(a.real < b.real)) && (!(a.real > b.real)) && (!(a.imag >= b.imag))) || isnan(a.imag))
                            : ((!(a.real <= b.real)) || ((!(a.real < b.real)) && (!(a.real > b.real)) && (!(a.imag <= b.imag))) || isnan(a.imag)));
         return take ? b : a;
      }
      else if constexpr ((EXTREME || ABSEXT) && (std::is_floating_point<Acc>::value))
      {  bool take = (!isnan(b)) && (ISMAX ? !(a >= b) : !(a <= b));
         return take ? b : a;
      }
      else return ISMAX ? ((a < b) ? b : a) : ((a > b) ? b : a);
   }

   /* ---- accumulator -> result ---- */
   static OCH_D Res finalize(Acc a, const Param &p)
   {
      if constexpr (LOGICAL) { obool r; r.v = a ? 1 : 0; return r; }
      else if constexpr (OP == R_NNZ || OP == R_NNZ_NAN) return a;
      else if constexpr (SUMLIKE)
      {  if constexpr (is_complex_v<T>)
         {  T r; r.real = from_work<E>((elemwork_t<T>)a.real); r.imag = from_work<E>((elemwork_t<T>)a.imag); return r; }
         else if constexpr (is_float_v<T>) return from_work<T>((W)a);
         else return a;
      }
      else if constexpr (ABSSUM)
      {  if constexpr (is_float_v<T> || is_complex_v<T>) return from_work<ABS>((typename traits<ABS>::work)a);
         else return a;
      }
      else if constexpr (EXTREME)
      {  if constexpr (is_bool_v<T>) { obool r; r.v = a; return r; }
         else if constexpr (is_complex_v<T>) { T r; r.real = from_work<E>(a.real); r.imag = from_work<E>(a.imag); return r; }
         else return from_work<T>(a);
      }
      else if constexpr (ABSEXT)
      {  if constexpr (is_bool_v<T>) { obool r; r.v = a; return r; }
         else if constexpr (is_int_v<T>) return a;
         else return from_work<ABS>(a);
      }
      else
      {  double v = (OP == R_NORM || OP == R_NORM_NAN) ? norm_pow(a, p.pinv) : sqrt(a);
         if constexpr (is_float_v<T> || is_complex_v<T>) return from_work<ABS>((typename traits<ABS>::work)v);
         else return v;
      }
   }
};

} /* namespace och */
