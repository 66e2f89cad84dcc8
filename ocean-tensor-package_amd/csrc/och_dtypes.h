/* Element types of the device library, their work types and the conversion
 * rules between them.
 *
 * Semantics restated from the reference (not its text):
 *   type list / order ......... solid/include/solid/base/generic/dtype_macros.h:133-147
 *   work types (half->float) .. solid/include/solid/base/gpu/dtype_gpu.h:83-85
 *   conversions ............... solid/include/solid/base/generic/dtype_assign.h:109-163,223-288
 *   software half ............. solid/src/base/generic/half.c:26-149
 *
 * Ocean's CPU module is the parity target, so half <-> float uses the CPU
 * routine's rounding (ties away from zero in magnitude, no subnormal results,
 * no special handling of the two boundary exponents) in integer arithmetic
 * instead of the hardware converters, and float -> integer conversion of
 * out-of-range values returns what the x86-64 scalar converters return.
 */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#define OCH_HD __host__ __device__ __forceinline__
#define OCH_D  __device__ __forceinline__

namespace och {

/* ---- storage types ---------------------------------------------------- */
struct obool   { uint8_t v; };
struct half_t  { uint16_t v; };
struct chalf_t { half_t real, imag; };
struct cfloat_t  { float  real, imag; };
struct cdouble_t { double real, imag; };

enum DTypeIndex {
   DT_BOOL = 0, DT_UINT8, DT_UINT16, DT_UINT32, DT_UINT64,
   DT_INT8, DT_INT16, DT_INT32, DT_INT64,
   DT_HALF, DT_FLOAT, DT_DOUBLE, DT_CHALF, DT_CFLOAT, DT_CDOUBLE, DT_COUNT
};

enum Kind { K_BOOL, K_UINT, K_SINT, K_FLOAT, K_COMPLEX };

template <class T> struct traits;
#define OCH_TRAITS(T, IDX, KIND, WORK, ELEM, ABS)                          \
   template <> struct traits<T> {                                          \
      static constexpr int  index = IDX;                                   \
      static constexpr Kind kind  = KIND;                                  \
      typedef WORK work;   /* type arithmetic is carried out in */         \
      typedef ELEM elem;   /* real/imag part type (self for real types) */ \
      typedef ABS  abs;    /* magnitude type */                            \
   };
OCH_TRAITS(obool,     DT_BOOL,    K_BOOL,    obool,     obool,    obool)
OCH_TRAITS(uint8_t,   DT_UINT8,   K_UINT,    uint8_t,   uint8_t,  uint8_t)
OCH_TRAITS(uint16_t,  DT_UINT16,  K_UINT,    uint16_t,  uint16_t, uint16_t)
OCH_TRAITS(uint32_t,  DT_UINT32,  K_UINT,    uint32_t,  uint32_t, uint32_t)
OCH_TRAITS(uint64_t,  DT_UINT64,  K_UINT,    uint64_t,  uint64_t, uint64_t)
OCH_TRAITS(int8_t,    DT_INT8,    K_SINT,    int8_t,    int8_t,   uint8_t)
OCH_TRAITS(int16_t,   DT_INT16,   K_SINT,    int16_t,   int16_t,  uint16_t)
OCH_TRAITS(int32_t,   DT_INT32,   K_SINT,    int32_t,   int32_t,  uint32_t)
OCH_TRAITS(int64_t,   DT_INT64,   K_SINT,    int64_t,   int64_t,  uint64_t)
OCH_TRAITS(half_t,    DT_HALF,    K_FLOAT,   float,     half_t,   half_t)
OCH_TRAITS(float,     DT_FLOAT,   K_FLOAT,   float,     float,    float)
OCH_TRAITS(double,    DT_DOUBLE,  K_FLOAT,   double,    double,   double)
OCH_TRAITS(chalf_t,   DT_CHALF,   K_COMPLEX, cfloat_t,  half_t,   half_t)
OCH_TRAITS(cfloat_t,  DT_CFLOAT,  K_COMPLEX, cfloat_t,  float,    float)
OCH_TRAITS(cdouble_t, DT_CDOUBLE, K_COMPLEX, cdouble_t, double,   double)
#undef OCH_TRAITS

template <class T> constexpr bool is_bool_v    = traits<T>::kind == K_BOOL;
template <class T> constexpr bool is_uint_v    = traits<T>::kind == K_UINT;
template <class T> constexpr bool is_sint_v    = traits<T>::kind == K_SINT;
template <class T> constexpr bool is_int_v     = is_uint_v<T> || is_sint_v<T>;
template <class T> constexpr bool is_float_v   = traits<T>::kind == K_FLOAT;
template <class T> constexpr bool is_complex_v = traits<T>::kind == K_COMPLEX;
template <class T> constexpr bool is_real_v    = !is_complex_v<T>;

/* ---- software half, Ocean CPU flavour ---------------------------------- */
OCH_HD float bits_to_float(uint32_t u) { union { uint32_t u; float f; } c; c.u = u; return c.f; }
OCH_HD uint32_t float_to_bits(float f) { union { uint32_t u; float f; } c; c.f = f; return c.u; }

/* The reference's routines in integer arithmetic, bit for bit (half.c:26-149): both zeros map to +0, subnormal halves
   are normalised, Inf / NaN keep their payload; float -> half returns zero below 2^-15, rounds ties (and above) up in
   magnitude with the carry running into the exponent, encodes the exponents 2^-15 and 2^16 as it does every other
   (which gives a subnormal pattern and a NaN pattern), and gives 0x7F00 for NaN. */
OCH_HD float half_to_float_soft(half_t hh)
{
   uint32_t h = hh.v;
   uint32_t s = (h & 0x8000u) << 16;
   h &= 0x7FFFu;
   if (h == 0) return 0.f;                       /* both zeros map to +0 */
   uint32_t e = h & 0x7C00u;
   if (e == 0)
   {  /* subnormal: normalise the mantissa */
      uint32_t shift = 1; h <<= 1;
      while (!(h & 0x0400u)) { shift++; h <<= 1; }
      h &= 0xFFFFu;                              /* the reference shifts a 16-bit variable */
      return bits_to_float(((h << 13) + ((112u - shift) << 23)) | s);
   }
   if (e == 0x7C00u) return bits_to_float((h << 13) | 0x7F800000u | s);
   return bits_to_float(((h << 13) + 0x38000000u) | s);
}

OCH_HD half_t float_to_half_soft(float f)
{
   uint32_t raw = float_to_bits(f);
   uint32_t d   = raw & 0x007FFFFFu;
   uint32_t s   = (raw >> 16) & 0x8000u;
   uint32_t ex  = (raw >> 23) & 0xFFu;
   half_t r;
   if (ex < 112u) { r.v = 0; return r; }
   if (ex > 143u)
   {  if (ex == 255u && d != 0) r.v = 0x7F00;    /* quiet NaN pattern 0x7F00, sign dropped */
      else r.v = (uint16_t)(s | 0x7C00u);
      return r;
   }
   uint32_t v = (((ex - 112u) << 10) | (d >> 13) | s) & 0xFFFFu;
   if ((d & 0x1FFFu) >= 0x1000u) v++;            /* ties round up in magnitude */
   r.v = (uint16_t)v;
   return r;
}

#if defined(__HIP_DEVICE_COMPILE__)
/* On the device the common case is a few instructions around the hardware converters, without a divergent branch:
   half -> float is exact in hardware for every value but a NaN (whose payload the integer routine carries over bit by
   bit), subnormals included, and adding +0 turns -0 into +0; float -> half with rounding toward zero gives, for
   2^-14 <= |f| < 2^16, exactly the reference's truncated pattern ((exponent - 112) << 10 | mantissa >> 13 | sign), to
   which the reference's rounding adds bit 12 of the float. Only lanes with a NaN half, or a float whose exponent is one
   of the two that the reference encodes in its own way or lies above them, take the integer routine -- behind a branch
   that is uniform over the wave, so waves without such a value never execute it. (The empty asm statements keep the
   compiler from turning those branches into unconditional arithmetic.) */
OCH_D float half_to_float(half_t hh)
{
   _Float16 x; __builtin_memcpy(&x, &hh.v, 2);
   float r = (float)x + 0.0f;
   if (__builtin_amdgcn_ballot_w64(r != r) != 0)
   {  asm volatile("" ::: "memory");
      if (r != r) r = bits_to_float(((uint32_t)(hh.v & 0x7FFFu) << 13) | 0x7F800000u | ((uint32_t)(hh.v & 0x8000u) << 16));
   }
   return r;
}
OCH_D half_t float_to_half(float f)
{
   const uint32_t raw = float_to_bits(f), a = raw & 0x7FFFFFFFu;
   const auto pk = __builtin_amdgcn_cvt_pkrtz(f, 0.0f);
   uint32_t t; __builtin_memcpy(&t, &pk, 4);
   const bool under = a < 0x38000000u;                               /* below 2^-15: zero, sign dropped */
   const uint32_t v = under ? 0u : t + ((raw >> 12) & 1u);
   /* exponent 2^-15, or 2^16 and above (values below 2^-15 are moved into the ordinary range for this test) */
   const uint32_t c = (under ? 0x38800000u : a) - 0x38800000u;
   half_t r; r.v = (uint16_t)v;
   if (__builtin_amdgcn_uicmp(c, 0x0F000000u, 35 /* unsigned >= : the lanes' results as one 64-bit mask */) != 0)
   {  asm volatile("" ::: "memory");
      if (c >= 0x0F000000u) r = float_to_half_soft(f);
   }
   return r;
}
#else
OCH_HD float half_to_float(half_t hh) { return half_to_float_soft(hh); }
OCH_HD half_t float_to_half(float f) { return float_to_half_soft(f); }
#endif

/* ---- float -> integer with x86-64 scalar converter results ------------- */
template <class F> OCH_HD int32_t cvtt_i32(F x)
{  /* cvttss2si/cvttsd2si r32: out of range or NaN -> 0x80000000 */
   if (x > (F)-2147483649.0 && x < (F)2147483648.0) return (int32_t)x;
   return (int32_t)0x80000000u;
}
template <> OCH_HD int32_t cvtt_i32<float>(float x)
{
   if (x >= -2147483648.0f && x < 2147483648.0f) return (int32_t)x;
   return (int32_t)0x80000000u;
}
template <class F> OCH_HD int64_t cvtt_i64(F x)
{  /* cvttss2si/cvttsd2si r64: out of range or NaN -> 0x8000000000000000 */
   if (x >= (F)-9223372036854775808.0 && x < (F)9223372036854775808.0) return (int64_t)x;
   return (int64_t)0x8000000000000000ull;
}
template <class F> OCH_HD uint64_t cvtt_u64(F x)
{  /* compiler sequence: values >= 2^63 are converted after subtracting 2^63 */
   if (x >= (F)9223372036854775808.0)
      return (uint64_t)cvtt_i64<F>(x - (F)9223372036854775808.0) ^ 0x8000000000000000ull;
   return (uint64_t)cvtt_i64<F>(x);
}

template <class I, class F> OCH_HD I float_to_int(F x)
{
   if constexpr (std::is_same<I, uint64_t>::value) return cvtt_u64<F>(x);
   else if constexpr (std::is_same<I, int64_t>::value)  return cvtt_i64<F>(x);
   else if constexpr (std::is_same<I, uint32_t>::value) return (uint32_t)cvtt_i64<F>(x);
   else return (I)cvtt_i32<F>(x);
}

/* ---- SOLID_CONVERT(TYPE1, TYPE2, X) for real (non-complex) types ------- */
template <class D, class S> OCH_HD D cvt_real(S x)
{
   if constexpr (std::is_same<D, S>::value) return x;
   else if constexpr (is_bool_v<D>)
   {  D r;
      if constexpr (std::is_same<S, half_t>::value) r.v = ((x.v & 0x7FFFu) == 0) ? 0 : 1;
      else r.v = (x == 0) ? 0 : 1;
      return r;
   }
   else if constexpr (is_bool_v<S>)
   {  if constexpr (std::is_same<D, half_t>::value) return float_to_half((float)x.v);
      else return (D)x.v;
   }
   else if constexpr (std::is_same<D, half_t>::value) return float_to_half((float)x);
   else if constexpr (std::is_same<S, half_t>::value) return cvt_real<D, float>(half_to_float(x));
   else if constexpr (is_int_v<D> && is_float_v<S>)   return float_to_int<D, S>(x);
   else return (D)x;
}

/* ---- SOLID_ASSIGN: any type to any type -------------------------------- */
template <class D, class S> OCH_HD D cvt(S x)
{
   if constexpr (std::is_same<D, S>::value) return x;
   else if constexpr (is_complex_v<S> && is_complex_v<D>)
   {  D r;
      r.real = cvt_real<typename traits<D>::elem>(x.real);
      r.imag = cvt_real<typename traits<D>::elem>(x.imag);
      return r;
   }
   else if constexpr (is_complex_v<S>)
   {  if constexpr (is_bool_v<D>)
      {  D r; r.v = (cvt_real<obool>(x.real).v || cvt_real<obool>(x.imag).v) ? 1 : 0; return r; }
      else return cvt_real<D>(x.real);
   }
   else if constexpr (is_complex_v<D>)
   {  D r;
      r.real = cvt_real<typename traits<D>::elem>(x);
      r.imag = cvt_real<typename traits<D>::elem>((uint8_t)0);
      return r;
   }
   else return cvt_real<D>(x);
}

/* To / from the work type (SOLID_TO_WORKTYPE / SOLID_FROM_WORKTYPE) */
template <class T> OCH_HD typename traits<T>::work to_work(T x)   { return cvt<typename traits<T>::work>(x); }
template <class T> OCH_HD T from_work(typename traits<T>::work x) { return cvt<T>(x); }

/* Work type of the real/imag part of a complex type */
template <class T> using elemwork_t = typename traits<typename traits<T>::elem>::work;

/* ---- byte reversal of each real part (SOLID_BYTESWAP) ------------------ */
OCH_HD uint16_t bswap16(uint16_t a) { return (uint16_t)((a << 8) | (a >> 8)); }
OCH_HD uint32_t bswap32(uint32_t a) { return __builtin_bswap32(a); }
OCH_HD uint64_t bswap64(uint64_t a) { return __builtin_bswap64(a); }

template <class T> OCH_HD T byteswap(T x)
{
   typedef typename traits<T>::elem E;
   if constexpr (sizeof(E) == 1) return x;
   else
   {  union U { T t; uint16_t h[8]; uint32_t w[4]; uint64_t q[2]; } u;
      u.t = x;
      constexpr int n = sizeof(T) / sizeof(E);
      if constexpr (sizeof(E) == 2) { for (int i = 0; i < n; i++) u.h[i] = bswap16(u.h[i]); }
      else if constexpr (sizeof(E) == 4) { for (int i = 0; i < n; i++) u.w[i] = bswap32(u.w[i]); }
      else { for (int i = 0; i < n; i++) u.q[i] = bswap64(u.q[i]); }
      return u.t;
   }
}

/* ---- dispatch helper: call f.template operator()<T>() for a dtype index */
#define OCH_FOR_ALL_TYPES(X) \
   X(obool) X(uint8_t) X(uint16_t) X(uint32_t) X(uint64_t) X(int8_t) X(int16_t) X(int32_t) X(int64_t) \
   X(half_t) X(float) X(double) X(chalf_t) X(cfloat_t) X(cdouble_t)

} /* namespace och */
