/* Binary elementwise operations z = f(x, y) for every element type.
 *
 * Semantics follow solid/include/solid/core/generic/binary_ops.h:112-520 and
 * the type table of solid/src/core/gpu/template_binary.cu:35-264:
 *   bool ...... + is OR, - is x & ~y, * and / are AND, mod is 0 (:115-136)
 *   integers .. wrap-around; x/0 = 0; signed divide and floor_divide round
 *               toward -inf; mod takes the sign of the divisor (:143-274)
 *   floats .... one IEEE operation in the work type (half works in float),
 *               min/max propagate NaN, fmin/fmax prefer non-NaN (:281-342)
 *   complex ... fixed operation order without fused multiply-add (:355-520)
 * Device code must be compiled with -ffp-contract=off so that no product is
 * fused into a following sum.
 */
#pragma once
#include "och_dtypes.h"
#include "och_math.h"
#include <math.h>

namespace och {

/* unsigned twin used to get wrap-around arithmetic without signed overflow */
template <class T> struct uwrap { typedef typename std::make_unsigned<T>::type type; };

template <class T> OCH_D T int_mul(T x, T y)
{  typedef typename uwrap<T>::type U;
   if constexpr (sizeof(T) < 4) return (T)((uint32_t)(U)x * (uint32_t)(U)y);
   else return (T)((U)x * (U)y);
}
template <class T> OCH_D T int_add(T x, T y)
{  typedef typename uwrap<T>::type U;
   if constexpr (sizeof(T) < 4) return (T)((uint32_t)(U)x + (uint32_t)(U)y);
   else return (T)((U)x + (U)y);
}
template <class T> OCH_D T int_sub(T x, T y)
{  typedef typename uwrap<T>::type U;
   if constexpr (sizeof(T) < 4) return (T)((uint32_t)(U)x - (uint32_t)(U)y);
   else return (T)((U)x - (U)y);
}

/* Sign test of the product x*y evaluated the way the reference evaluates it:
   in `int` for 8/16-bit operands, in the operand type (wrapping) otherwise. */
template <class T> OCH_D bool prod_negative(T x, T y)
{
   if constexpr (sizeof(T) < 4) return ((int32_t)x * (int32_t)y) < 0;
   else return int_mul<T>(x, y) < 0;
}

/* magnitude of a signed value as its unsigned twin (the most negative value keeps its bit pattern, 2^(bits-1)) */
template <class T> OCH_D typename uwrap<T>::type int_magnitude(T x)
{  typedef typename uwrap<T>::type U; return (x < 0) ? (U)((U)0 - (U)x) : (U)x; }

/* Quotient of the reference's integer expressions, evaluated in `int` for
   8/16-bit operands (so -128 / -1 wraps on the final store only). 64-bit signed operands divide as magnitudes: the
   unsigned division takes its short form (one 32-bit division) whenever both magnitudes fit 32 bits -- the signed one
   only when both operands are non-negative, so mixed signs in a wave ran the short and the long form one after the other
   -- and the most negative value divided by -1 comes out wrapped without a case of its own. */
template <class T> OCH_D T int_quot(T x, T y)
{
   if constexpr (is_uint_v<T>) return (T)(x / y);
   else if constexpr (sizeof(T) < 4) return (T)((int32_t)x / (int32_t)y);
   else if constexpr (sizeof(T) == 8)
   {  typedef typename uwrap<T>::type U;
      const U q = int_magnitude<T>(x) / int_magnitude<T>(y);
      return (T)(((x < 0) != (y < 0)) ? (U)((U)0 - q) : q);
   }
   else
   {  /* most-negative / -1 overflows; the x86 result the CPU path would trap on is not
         reproducible, return the wrapped value */
      if (y == (T)-1) return int_sub<T>((T)0, x);
      return (T)(x / y);
   }
}
template <class T> OCH_D T int_rem(T x, T y)
{
   if constexpr (is_uint_v<T>) return (T)(x % y);
   else if constexpr (sizeof(T) < 4) return (T)((int32_t)x % (int32_t)y);
   else if constexpr (sizeof(T) == 8)
   {  /* the remainder takes the sign of the dividend; x % -1 = 0 follows */
      typedef typename uwrap<T>::type U;
      const U r = int_magnitude<T>(x) % int_magnitude<T>(y);
      return (T)((x < 0) ? (U)((U)0 - r) : r);
   }
   else { if (y == (T)-1) return (T)0; return (T)(x % y); }
}

#define OCH_BINARY_TYPES(TA, TB, TR) typedef TA A; typedef TB B; typedef TR R;

/* ------------------------------------------------------------------------ */
template <class T> struct BinAdd
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = x.v | y.v; return z; }
      else if constexpr (is_int_v<T>) return int_add<T>(x, y);
      else if constexpr (is_float_v<T>) return from_work<T>(to_work(x) + to_work(y));
      else
      {  typedef typename traits<T>::elem E; R z;
         z.real = from_work<E>(to_work(x.real) + to_work(y.real));
         z.imag = from_work<E>(to_work(x.imag) + to_work(y.imag));
         return z;
      }
   }
};

template <class T> struct BinSubtract
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = x.v & (uint8_t)~y.v; return z; }
      else if constexpr (is_int_v<T>) return int_sub<T>(x, y);
      else if constexpr (is_float_v<T>) return from_work<T>(to_work(x) - to_work(y));
      else
      {  typedef typename traits<T>::elem E; R z;
         z.real = from_work<E>(to_work(x.real) - to_work(y.real));
         z.imag = from_work<E>(to_work(x.imag) - to_work(y.imag));
         return z;
      }
   }
};

template <class T> struct BinMultiply
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = x.v & y.v; return z; }
      else if constexpr (is_int_v<T>) return int_mul<T>(x, y);
      else if constexpr (is_float_v<T>) return from_work<T>(to_work(x) * to_work(y));
      else
      {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W; R z;
         W xr = to_work(x.real), xi = to_work(x.imag), yr = to_work(y.real), yi = to_work(y.imag);
         z.real = from_work<E>(xr * yr - xi * yi);
         z.imag = from_work<E>(xr * yi + yr * xi);
         return z;
      }
   }
};

template <class T> struct BinTrueDivide
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = x.v & y.v; return z; }
      else if constexpr (is_int_v<T>) return (y == 0) ? (T)0 : int_quot<T>(x, y);
      else if constexpr (is_float_v<T>) return from_work<T>(to_work(x) / to_work(y));
      else
      {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W; R z;
         W xr = to_work(x.real), xi = to_work(x.imag), yr = to_work(y.real), yi = to_work(y.imag);
         W r = yr * yr + yi * yi;
         z.real = from_work<E>((xr * yr + xi * yi) / r);
         z.imag = from_work<E>((xi * yr - xr * yi) / r);
         return z;
      }
   }
};

/* Signed division rounding toward -inf: x is moved by (y -/+ 1) when the signs differ,
   then divided. For 8/16-bit operands the reference evaluates `divide` entirely in `int`
   (:178) while `floor_divide` stores the adjusted x back into the operand type first
   (:200-201); TRUNC selects the second behaviour. */
template <class T, bool TRUNC> OCH_D T int_floor_div(T x, T y)
{
   if (y == 0) return (T)0;
   if constexpr (sizeof(T) < 4)
   {  int32_t xx = x, yy = y;
      xx -= ((xx * yy) < 0) * (yy + ((yy < 0) - (yy > 0)));
      if constexpr (TRUNC) xx = (T)xx;
      return (T)(xx / yy);
   }
   else
   {  T adj = (T)(prod_negative<T>(x, y) ? int_add<T>(y, (T)((y < 0) - (y > 0))) : (T)0);
      return int_quot<T>(int_sub<T>(x, adj), y);
   }
}

template <class T> struct BinDivide
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_sint_v<T>) return int_floor_div<T, false>(x, y);
      else return BinTrueDivide<T>::f(x, y);
   }
};

template <class T> struct BinFloorDivide   /* not defined for complex */
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_sint_v<T>) return int_floor_div<T, true>(x, y);
      else if constexpr (is_float_v<T>)
      {  typedef typename traits<T>::work W; W a = to_work(x), b = to_work(y);
         return from_work<T>((W)floor(a / b));
      }
      else return BinTrueDivide<T>::f(x, y);
   }
};

template <class T> struct BinMod           /* not defined for complex */
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = 0; return z; }
      else if constexpr (is_uint_v<T>) return (y == 0) ? (T)0 : (T)(x % y);
      else if constexpr (is_sint_v<T>)
      {  if (y == 0) return (T)0;
         T z = int_rem<T>(x, y);
         return (T)((prod_negative<T>(x, y) && (z != 0)) ? int_add<T>(z, y) : z);
      }
      else
      {  typedef typename traits<T>::work W; W a = to_work(x), b = to_work(y);
         W q = (W)floor(a / b);
         return from_work<T>(a - q * b);
      }
   }
};

template <class T> struct BinFMod          /* not defined for complex */
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = 0; return z; }
      else if constexpr (is_int_v<T>) return (y == 0) ? (T)0 : int_rem<T>(x, y);
      else
      {  typedef typename traits<T>::work W; W a = to_work(x), b = to_work(y);
         return from_work<T>((W)fmod((double)a, (double)b));
      }
   }
};

/* power: integer and bool bases take an int16 exponent */
template <class T> struct BinPower
{  typedef T A; typedef T R;
   typedef typename std::conditional<(is_bool_v<T> || is_int_v<T>), int16_t, T>::type B;
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = ((x.v != 0) | (y == 0)) ? 1 : 0; return z; }
      else if constexpr (is_int_v<T>)
      {  T b = x, z; int64_t e = y;
         z = (T)(e >= 0);
         while (e > 0) { if (e & 1) z = int_mul<T>(z, b); e >>= 1; b = int_mul<T>(b, b); }
         return z;
      }
      else if constexpr (std::is_same<T, double>::value)
         return (double)och_powf((float)x, (float)y);   /* the CPU path evaluates double pow in single precision */
      else if constexpr (is_float_v<T>) return from_work<T>(och_powf(to_work(x), to_work(y)));
      else
      {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W; R z;
         W xr = to_work(x.real), xi = to_work(x.imag), yr = to_work(y.real), yi = to_work(y.imag);
         W scale = xr * xr + xi * xi, zr, zi;
         if (scale == 0)
         {  z.real = from_work<E>((W)((yr == 0) && (yi == 0)));
            z.imag = cvt_real<E>((uint8_t)0);
            return z;
         }
         if constexpr (std::is_same<W, float>::value)
         {  zi = atan2f(xi, xr); zr = (W)(logf(scale) * 0.5);
            xr = yr * zr - yi * zi; xi = yr * zi + yi * zr;
            W sn, cs; sincosf(xi, &sn, &cs);          /* one argument reduction for both */
            scale = expf(xr); xr = scale * cs; xi = scale * sn;
         }
         else
         {  zi = atan2(xi, xr); zr = log(scale) * 0.5;
            xr = yr * zr - yi * zi; xi = yr * zi + yi * zr;
            W sn, cs; sincos(xi, &sn, &cs);
            scale = exp(xr); xr = scale * cs; xi = scale * sn;
         }
         z.real = from_work<E>(xr); z.imag = from_work<E>(xi);
         return z;
      }
   }
};

/* ---- min / max ---------------------------------------------------------- */
template <class T, bool MAX, bool F> struct BinMinMax
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = MAX ? (x.v | y.v) : (x.v & y.v); return z; }
      else if constexpr (is_int_v<T>) { if constexpr (MAX) return (x >= y) ? x : y; else return (x <= y) ? x : y; }
      else if constexpr (is_float_v<T>)
      {  typedef typename traits<T>::work W; W a = to_work(x), b = to_work(y);
         if constexpr (!F) { if (isnan(b) || (MAX ? (b > a) : (b < a))) a = b; }     /* NaN propagates */
         else              { if (isnan(a) || (MAX ? (b >= a) : (b <= a))) a = b; }   /* NaN avoided */
         return from_work<T>(a);
      }
      else
      {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W; R z;
         W xr = to_work(x.real), xi = to_work(x.imag), yr = to_work(y.real), yi = to_work(y.imag);
         bool take;
         if constexpr (!F)
            take = (isnan(yr) || isnan(yi)) || (MAX ? (yr > xr) : (yr < xr)) ||
                   ((yr == xr) && (MAX ? (yi > xi) : (yi < xi)));
         else
            take = ((MAX ? (yr > xr) : (yr < xr)) || isnan(xr)) ||
                   ((xr == yr) && ((MAX ? (yi > xi) : (yi < xi)) || isnan(xi)));
         z.real = from_work<E>(take ? yr : xr);
         z.imag = from_work<E>(take ? yi : xi);
         return z;
      }
   }
};
template <class T> using BinMin  = BinMinMax<T, false, false>;
template <class T> using BinMax  = BinMinMax<T, true,  false>;
template <class T> using BinFMin = BinMinMax<T, false, true>;
template <class T> using BinFMax = BinMinMax<T, true,  true>;

/* ---- comparisons: result is bool; complex compares lexicographically ---- */
enum CmpKind { CMP_LT, CMP_LE, CMP_EQ, CMP_NE, CMP_GE, CMP_GT };
template <class W, int C> OCH_D bool cmp_scalar(W a, W b)
{
   if constexpr (C == CMP_LT) return a < b;
   else if constexpr (C == CMP_LE) return a <= b;
   else if constexpr (C == CMP_EQ) return a == b;
   else if constexpr (C == CMP_NE) return a != b;
   else if constexpr (C == CMP_GE) return a >= b;
   else return a > b;
}
template <class T, int C> struct BinCompare
{  OCH_BINARY_TYPES(T, T, obool)
   static OCH_D R f(A x, B y)
   {  R z;
      if constexpr (is_bool_v<T>) z.v = cmp_scalar<uint8_t, C>(x.v, y.v) ? 1 : 0;
      else if constexpr (is_int_v<T>) z.v = cmp_scalar<T, C>(x, y) ? 1 : 0;
      else if constexpr (is_float_v<T>) z.v = cmp_scalar<typename traits<T>::work, C>(to_work(x), to_work(y)) ? 1 : 0;
      else
      {  typedef elemwork_t<T> W;
         W xr = to_work(x.real), xi = to_work(x.imag), yr = to_work(y.real), yi = to_work(y.imag);
         if constexpr (C == CMP_EQ) z.v = ((xr == yr) && (xi == yi)) ? 1 : 0;
         else if constexpr (C == CMP_NE) z.v = ((xr != yr) || (xi != yi)) ? 1 : 0;
         else if constexpr (C == CMP_LT) z.v = (xr != yr) ? (xr < yr) : (xi <  yi);
         else if constexpr (C == CMP_LE) z.v = (xr != yr) ? (xr < yr) : (xi <= yi);
         else if constexpr (C == CMP_GE) z.v = (xr != yr) ? (xr > yr) : (xi >= yi);
         else                            z.v = (xr != yr) ? (xr > yr) : (xi >  yi);
      }
      return z;
   }
};
template <class T> using BinLT = BinCompare<T, CMP_LT>;
template <class T> using BinLE = BinCompare<T, CMP_LE>;
template <class T> using BinEQ = BinCompare<T, CMP_EQ>;
template <class T> using BinNE = BinCompare<T, CMP_NE>;
template <class T> using BinGE = BinCompare<T, CMP_GE>;
template <class T> using BinGT = BinCompare<T, CMP_GT>;

/* ---- bitwise / logical (bool and integers) ------------------------------ */
template <class T, int OP> struct BinBit     /* 0: and, 1: or, 2: xor */
{  OCH_BINARY_TYPES(T, T, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>)
      {  R z; z.v = (OP == 0) ? (x.v & y.v) : (OP == 1) ? (x.v | y.v) : (x.v ^ y.v); return z; }
      else return (T)((OP == 0) ? (x & y) : (OP == 1) ? (x | y) : (x ^ y));
   }
};
template <class T> using BinBitAnd = BinBit<T, 0>;
template <class T> using BinBitOr  = BinBit<T, 1>;
template <class T> using BinBitXor = BinBit<T, 2>;

/* Shifts: the count is an int8; a negative count shifts the other way. 8/16-bit
   operands are shifted as 32-bit integers and truncated on store; counts are
   taken modulo the register width like the x86 shifters do. */
template <class T> OCH_D T shift_left(T x, int c)
{
   if constexpr (sizeof(T) < 8)
   {  if constexpr (is_sint_v<T>) return (T)((uint32_t)(int32_t)x << (c & 31));
      else return (T)((uint32_t)x << (c & 31));
   }
   else return (T)((uint64_t)x << (c & 63));
}
template <class T> OCH_D T shift_right(T x, int c)
{
   if constexpr (sizeof(T) < 8)
   {  if constexpr (is_sint_v<T>) return (T)((int32_t)x >> (c & 31));
      else return (T)((uint32_t)x >> (c & 31));
   }
   else
   {  if constexpr (is_sint_v<T>) return (T)((int64_t)x >> (c & 63));
      else return (T)((uint64_t)x >> (c & 63));
   }
}
template <class T, bool LEFT> struct BinShift
{  OCH_BINARY_TYPES(T, int8_t, T)
   static OCH_D R f(A x, B y)
   {  if constexpr (is_bool_v<T>) { R z; z.v = (y == 0) ? (x.v & 1) : 0; return z; }
      else
      {  int s = y;
         if (LEFT) return (s < 0) ? shift_right<T>(x, -s) : shift_left<T>(x, s);
         else      return (s < 0) ? shift_left<T>(x, -s)  : shift_right<T>(x, s);
      }
   }
};
template <class T> using BinShiftLeft  = BinShift<T, true>;
template <class T> using BinShiftRight = BinShift<T, false>;

} /* namespace och */
