/* TEST INFRASTRUCTURE -- CPU restatement of Ocean's Solid CPU semantics.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may use
 * anything in this directory; the product never links or loads it.
 *
 * Element types, software half precision and conversions, restated from
 *   solid/include/solid/base/generic/dtype_macros.h:133-173 (type list),
 *   solid/include/solid/base/cpu/dtype_cpu.h:27-80 (work types, special conversions),
 *   solid/include/solid/base/generic/dtype_assign.h:109-163,223-288 (SOLID_CONVERT / SOLID_ASSIGN),
 *   solid/src/base/generic/half.c:26-149 (half <-> float).
 * Pinned by tests/test_oracle_ref.py against the reference's own half.c and
 * conversion macros compiled into oracle/_ref (exhaustive over all 65536 halves,
 * sampled floats including ties and range boundaries, all 15x15 type pairs).
 */
#ifndef ORACLE_TYPES_H
#define ORACLE_TYPES_H

#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>

typedef uint8_t  o_bool;
typedef uint16_t o_half;
typedef struct { o_half real, imag; } o_chalf;
typedef struct { float  real, imag; } o_cfloat;
typedef struct { double real, imag; } o_cdouble;

enum { O_BOOL = 0, O_UINT8, O_UINT16, O_UINT32, O_UINT64, O_INT8, O_INT16, O_INT32, O_INT64,
       O_HALF, O_FLOAT, O_DOUBLE, O_CHALF, O_CFLOAT, O_CDOUBLE, O_NTYPES };

static const int o_type_size[O_NTYPES] = { 1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 4, 8, 16 };

#define O_MAX_DIMS 8

/* ---- half precision (half.c:26-149) ------------------------------------ */
static inline float o_half_to_float(o_half h)
{
   uint32_t sign = ((uint32_t)(h & 0x8000)) << 16, bits;
   float f;
   h &= 0x7FFF;
   if (h == 0) return 0.f;
   if ((h & 0x7C00) == 0)
   {  /* subnormal half: shift until the leading one reaches bit 10 */
      uint32_t n = 1;
      h = (o_half)(h << 1);
      while ((h & 0x0400) == 0) { n++; h = (o_half)(h << 1); }
      bits = (((uint32_t)h) << 13) + ((112 - n) << 23);
   }
   else if ((h & 0x7C00) == 0x7C00) bits = (((uint32_t)h) << 13) | 0x7F800000u;
   else bits = (((uint32_t)h) << 13) + 0x38000000u;
   bits |= sign;
   memcpy(&f, &bits, 4);
   return f;
}

static inline o_half o_float_to_half(float f)
{
   uint32_t raw, mant;
   uint16_t sign, e;
   memcpy(&raw, &f, 4);
   mant = raw & 0x007FFFFFu;
   e = (uint16_t)(raw >> 16);
   sign = e & 0x8000;
   e = (uint16_t)((e & 0x7FFF) >> 7);
   if (e < 127 - 15) return 0;                       /* zero and underflow */
   if (e > 127 + 16)
   {  if (e == 255 && mant != 0) return 0x7F00;      /* NaN (the quiet-NaN pattern of half.h:26) */
      return (o_half)(sign | 0x7C00);                /* infinity and overflow */
   }
   e = (uint16_t)(e - (127 - 15));
   e = (uint16_t)(e << 10);
   e |= (uint16_t)(mant >> 13);
   e |= sign;
   if ((mant & 0x1FFF) >= 0x1000) e++;
   return e;
}

#endif
