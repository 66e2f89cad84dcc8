/* TEST INFRASTRUCTURE (see oracle_types.h).
 * Value conversions between the 15 element types, restated from
 * solid/include/solid/base/generic/dtype_assign.h:109-163 (SOLID_CONVERT),
 * :223-288 (SOLID_ASSIGN), :55-83,171-214 (SOLID_BYTESWAP) and the special-type
 * rules of solid/include/solid/base/cpu/dtype_cpu.h:68-80.
 *   basic -> basic ........ C cast
 *   anything -> bool ...... value != 0 (half: any bit below the sign)
 *   basic <-> half ........ through float with the software converter
 *   complex -> real ....... real part;  real -> complex: imaginary part 0
 *   complex -> bool ....... real != 0 || imag != 0
 */
#ifndef ORACLE_CONVERT_H
#define ORACLE_CONVERT_H
#include "oracle_types.h"

typedef o_bool   o_t_bool;
typedef uint8_t  o_t_uint8;   typedef uint16_t o_t_uint16; typedef uint32_t o_t_uint32; typedef uint64_t o_t_uint64;
typedef int8_t   o_t_int8;    typedef int16_t  o_t_int16;  typedef int32_t  o_t_int32;  typedef int64_t  o_t_int64;
typedef o_half   o_t_half;    typedef float    o_t_float;  typedef double   o_t_double;
typedef o_chalf  o_t_chalf;   typedef o_cfloat o_t_cfloat; typedef o_cdouble o_t_cdouble;

/* kind of a real type: B bool, H half, N native C arithmetic type */
#define O_KIND_bool B
#define O_KIND_uint8 N
#define O_KIND_uint16 N
#define O_KIND_uint32 N
#define O_KIND_uint64 N
#define O_KIND_int8 N
#define O_KIND_int16 N
#define O_KIND_int32 N
#define O_KIND_int64 N
#define O_KIND_half H
#define O_KIND_float N
#define O_KIND_double N

#define O_CVT_N_N(S, D, x) ((o_t_##D)(x))
#define O_CVT_N_B(S, D, x) ((((o_t_##S)(x)) == 0) ? 0 : 1)
#define O_CVT_N_H(S, D, x) o_float_to_half((float)(x))
#define O_CVT_B_N(S, D, x) ((o_t_##D)(x))
#define O_CVT_B_B(S, D, x) (x)
#define O_CVT_B_H(S, D, x) o_float_to_half((float)(x))
#define O_CVT_H_N(S, D, x) ((o_t_##D)o_half_to_float(x))
#define O_CVT_H_B(S, D, x) ((((x) & 0x7FFF) == 0) ? 0 : 1)
#define O_CVT_H_H(S, D, x) (x)
#define O_CVT3(SK, DK, S, D, x) O_CVT_##SK##_##DK(S, D, x)
#define O_CVT2(SK, DK, S, D, x) O_CVT3(SK, DK, S, D, x)

#define O_REAL_TYPES(M, A) \
   M(A, bool) M(A, uint8) M(A, uint16) M(A, uint32) M(A, uint64) \
   M(A, int8) M(A, int16) M(A, int32) M(A, int64) M(A, half) M(A, float) M(A, double)

#define O_REAL_TYPES_INNER(M, A) \
   M(A, bool) M(A, uint8) M(A, uint16) M(A, uint32) M(A, uint64) \
   M(A, int8) M(A, int16) M(A, int32) M(A, int64) M(A, half) M(A, float) M(A, double)

/* o_cvt_<src>_<dst>(x) for the 12 x 12 real pairs */
#define O_DEF_CVT(S, D) \
   static inline o_t_##D o_cvt_##S##_##D(o_t_##S x) { return O_CVT2(O_KIND_##S, O_KIND_##D, S, D, x); }
#define O_DEF_CVT_ROW(A, S) O_REAL_TYPES_INNER(O_DEF_CVT_SWAP, S)
#define O_DEF_CVT_SWAP(S, D) O_DEF_CVT(S, D)
O_REAL_TYPES(O_DEF_CVT_ROW, _)

/* byte reversal of one real value */
static inline uint16_t o_swap16(uint16_t a) { return (uint16_t)(((a & 0x00FF) << 8) | ((a & 0xFF00) >> 8)); }
static inline uint32_t o_swap32(uint32_t a)
{  return ((a & 0x000000FFu) << 24) | ((a & 0x0000FF00u) << 8) | ((a & 0x00FF0000u) >> 8) | ((a & 0xFF000000u) >> 24); }
static inline uint64_t o_swap64(uint64_t a)
{  return ((uint64_t)o_swap32((uint32_t)(a & 0xFFFFFFFFu)) << 32) | (uint64_t)o_swap32((uint32_t)(a >> 32)); }

/* reverse the bytes of `n` consecutive parts of `width` bytes, src -> dst (may alias) */
static inline void o_swap_parts(const void *src, void *dst, int width, int n)
{
   int i;
   for (i = 0; i < n; i++)
   {  const char *s = (const char *)src + i * width; char *d = (char *)dst + i * width;
      if (width == 1) { *d = *s; }
      else if (width == 2) { uint16_t v; memcpy(&v, s, 2); v = o_swap16(v); memcpy(d, &v, 2); }
      else if (width == 4) { uint32_t v; memcpy(&v, s, 4); v = o_swap32(v); memcpy(d, &v, 4); }
      else { uint64_t v; memcpy(&v, s, 8); v = o_swap64(v); memcpy(d, &v, 8); }
   }
}

/* width of a real part and number of parts per element */
static const int o_part_size[O_NTYPES]  = { 1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 2, 4, 8 };
static const int o_part_count[O_NTYPES] = { 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 2 };

#endif
