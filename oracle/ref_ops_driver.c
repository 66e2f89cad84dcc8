/* TEST INFRASTRUCTURE -- builds oracle/_ref/libocean_ref.so from the REFERENCE'S OWN
 * headers where they lie under /root/reference (nothing is copied into this repository).
 *
 * The reference's CPU kernel sources (solid/src/core/cpu/template_*.c) cannot be built
 * here: they need solid_omp_config.h, which cmake generates, and the reductions also need
 * solid_core_cpu.h, which solid/bin/generate.py writes. What does compile from plain source
 * is the arithmetic itself: the operation macros of solid/include/solid/core/generic/
 * {binary_ops.h,unary_ops.h,reduce_ops.h}, the conversion macros of
 * solid/include/solid/base/generic/dtype_assign.h and solid/src/base/generic/half.c.
 * This driver instantiates those macros for every element type inside plain contiguous
 * loops of its own and exports them through small tables, so that the restated oracle can
 * be checked element by element against the reference text compiled by the same compiler.
 * The per-type expansion uses the reference's own generate_all_types.h mechanism.
 */
#ifndef SD_TEMPLATE_FILE
#define SD_TEMPLATE_FILE "ref_ops_driver.c"

#include <stddef.h>
#include <stdint.h>
#include "solid/base/generic/dtype_macros.h"
#include "solid/base/generic/dtype_assign.h"
#include "solid/base/cpu/dtype_cpu.h"
#include "solid/base/generic/generate_macros.h"

#define REF_CAT_(a, b) a##_##b
#define REF_CAT(a, b) REF_CAT_(a, b)

typedef void (*ref_bin_fn)(size_t n, const void *x, const void *y, void *z);
typedef void (*ref_un_fn)(size_t n, const void *x, void *y);
typedef void (*ref_red_fn)(size_t n, const void *x, const void *prm, void *result);

enum { RB_ADD, RB_SUBTRACT, RB_MULTIPLY, RB_DIVIDE, RB_TRUE_DIVIDE, RB_FLOOR_DIVIDE, RB_POWER, RB_MOD, RB_FMOD,
       RB_MIN, RB_MAX, RB_FMIN, RB_FMAX, RB_LT, RB_LE, RB_EQ, RB_NE, RB_GE, RB_GT,
       RB_BITAND, RB_BITOR, RB_BITXOR, RB_LAND, RB_LOR, RB_LXOR, RB_SHL, RB_SHR, RB_COUNT };
enum { RU_NEGATIVE, RU_BITNOT, RU_LNOT, RU_CONJ, RU_RECIPROCAL, RU_SIN, RU_COS, RU_TAN, RU_SINH, RU_COSH, RU_TANH,
       RU_ARCSIN, RU_ARCCOS, RU_ARCTAN, RU_ARCSINH, RU_ARCCOSH, RU_ARCTANH, RU_SQRT, RU_CBRT, RU_SQUARE,
       RU_EXP, RU_EXP2, RU_EXP10, RU_EXPM1, RU_LOG, RU_LOG2, RU_LOG10, RU_LOG1P, RU_ABSOLUTE, RU_FABS, RU_SIGN,
       RU_CEIL, RU_FLOOR, RU_TRUNC, RU_ROUND, RU_ISINF, RU_ISNAN, RU_ISFINITE, RU_ISPOSINF, RU_ISNEGINF, RU_COUNT };
enum { RR_ANY, RR_ALL, RR_ALL_FINITE, RR_ANY_INF, RR_ANY_NAN, RR_NNZ, RR_NNZ_NAN,
       RR_ALL_LT, RR_ALL_LE, RR_ALL_GT, RR_ALL_GE, RR_ALL_GTLT, RR_ALL_GTLE, RR_ALL_GELT, RR_ALL_GELE,
       RR_SUM, RR_SUM_NAN, RR_PROD, RR_PROD_NAN, RR_SUM_ABS, RR_SUM_ABS_NAN,
       RR_MAXIMUM, RR_MINIMUM, RR_MAXIMUM_ABS, RR_MINIMUM_ABS, RR_NORM, RR_NORM_NAN, RR_NORM2, RR_NORM2_NAN, RR_COUNT };

static ref_bin_fn ref_bin_table[RB_COUNT][15];
static ref_un_fn  ref_un_table[RU_COUNT][15];
static ref_red_fn ref_red_table[RR_COUNT][15];

ref_bin_fn ref_binary(int op, int dtype) { return (op >= 0 && op < RB_COUNT && dtype >= 0 && dtype < 15) ? ref_bin_table[op][dtype] : 0; }
ref_un_fn  ref_unary(int op, int dtype)  { return (op >= 0 && op < RU_COUNT && dtype >= 0 && dtype < 15) ? ref_un_table[op][dtype] : 0; }
ref_red_fn ref_reduce(int op, int dtype) { return (op >= 0 && op < RR_COUNT && dtype >= 0 && dtype < 15) ? ref_red_table[op][dtype] : 0; }

float    ref_half_to_float(uint16_t h) { return solid_half_to_float(h); }
uint16_t ref_float_to_half(float f)    { return solid_float_to_half(f); }

#include "solid/base/generic/generate_all_types.h"

#else  /* ---------------- per-type section: SDXTYPE is defined ---------------- */

#include "solid/core/cpu/binary_ops_cpu.h"     /* defines SOLID_OP_<binary> and SOLID_OP_<unary> for SDXTYPE */

#define REF_T  SOLID_C_TYPE(SDXTYPE)
#define REF_IDX SDTYPE_INDEX(SDXTYPE)

/* ---- binary ---- */
#define REF_BIN(NAME, ID, OP, TY, TZ)                                                        \
   static void REF_CAT(REF_CAT(refb, NAME), SDXTYPE)(size_t n, const void *x, const void *y, void *z) \
   {  const REF_T *px = (const REF_T *)x; const SOLID_C_TYPE(TY) *py = (const SOLID_C_TYPE(TY) *)y;   \
      SOLID_C_TYPE(TZ) *pz = (SOLID_C_TYPE(TZ) *)z; size_t i;                                \
      for (i = 0; i < n; i++) { OP(px[i], py[i], pz[i]) }                                    \
   }                                                                                         \
   __attribute__((constructor)) static void REF_CAT(REF_CAT(regb, NAME), SDXTYPE)(void)      \
   {  ref_bin_table[ID][REF_IDX] = REF_CAT(REF_CAT(refb, NAME), SDXTYPE); }

REF_BIN(add, RB_ADD, SOLID_OP_ADD, SDXTYPE, SDXTYPE)
REF_BIN(subtract, RB_SUBTRACT, SOLID_OP_SUBTRACT, SDXTYPE, SDXTYPE)
REF_BIN(multiply, RB_MULTIPLY, SOLID_OP_MULTIPLY, SDXTYPE, SDXTYPE)
REF_BIN(true_divide, RB_TRUE_DIVIDE, SOLID_OP_TRUE_DIVIDE, SDXTYPE, SDXTYPE)
REF_BIN(divide, RB_DIVIDE, SOLID_OP_DIVIDE, SDXTYPE, SDXTYPE)
#if (!SDTYPE_IS_BOOL(SDXTYPE))
REF_BIN(min, RB_MIN, SOLID_OP_MIN, SDXTYPE, SDXTYPE)
REF_BIN(max, RB_MAX, SOLID_OP_MAX, SDXTYPE, SDXTYPE)
REF_BIN(fmin, RB_FMIN, SOLID_OP_FMIN, SDXTYPE, SDXTYPE)
REF_BIN(fmax, RB_FMAX, SOLID_OP_FMAX, SDXTYPE, SDXTYPE)
#endif
#if (!SDTYPE_IS_COMPLEX(SDXTYPE))
REF_BIN(mod, RB_MOD, SOLID_OP_MOD, SDXTYPE, SDXTYPE)
REF_BIN(fmod, RB_FMOD, SOLID_OP_FMOD, SDXTYPE, SDXTYPE)
REF_BIN(floor_divide, RB_FLOOR_DIVIDE, SOLID_OP_FLOOR_DIVIDE, SDXTYPE, SDXTYPE)
#endif
#if (SDTYPE_IS_BOOL(SDXTYPE) || SDTYPE_IS_INT(SDXTYPE))
REF_BIN(bitand, RB_BITAND, SOLID_OP_BITAND, SDXTYPE, SDXTYPE)
REF_BIN(bitor, RB_BITOR, SOLID_OP_BITOR, SDXTYPE, SDXTYPE)
REF_BIN(bitxor, RB_BITXOR, SOLID_OP_BITXOR, SDXTYPE, SDXTYPE)
REF_BIN(shl, RB_SHL, SOLID_OP_BITSHIFT_LEFT, int8, SDXTYPE)
REF_BIN(shr, RB_SHR, SOLID_OP_BITSHIFT_RIGHT, int8, SDXTYPE)
REF_BIN(power, RB_POWER, SOLID_OP_POWER, int16, SDXTYPE)
#else
REF_BIN(power, RB_POWER, SOLID_OP_POWER, SDXTYPE, SDXTYPE)
#endif
#if (SDTYPE_IS_BOOL(SDXTYPE))
REF_BIN(land, RB_LAND, SOLID_OP_BITAND, SDXTYPE, SDXTYPE)
REF_BIN(lor, RB_LOR, SOLID_OP_BITOR, SDXTYPE, SDXTYPE)
REF_BIN(lxor, RB_LXOR, SOLID_OP_BITXOR, SDXTYPE, SDXTYPE)
#endif
REF_BIN(lt, RB_LT, SOLID_OP_LT, SDXTYPE, bool)
REF_BIN(le, RB_LE, SOLID_OP_LE, SDXTYPE, bool)
REF_BIN(eq, RB_EQ, SOLID_OP_EQ, SDXTYPE, bool)
REF_BIN(ne, RB_NE, SOLID_OP_NE, SDXTYPE, bool)
REF_BIN(ge, RB_GE, SOLID_OP_GE, SDXTYPE, bool)
REF_BIN(gt, RB_GT, SOLID_OP_GT, SDXTYPE, bool)

/* ---- unary ---- */
#define REF_UN(NAME, ID, OP, TY)                                                             \
   static void REF_CAT(REF_CAT(refu, NAME), SDXTYPE)(size_t n, const void *x, void *y)       \
   {  const REF_T *px = (const REF_T *)x; SOLID_C_TYPE(TY) *py = (SOLID_C_TYPE(TY) *)y; size_t i; \
      for (i = 0; i < n; i++) { OP(px[i], py[i]) }                                           \
   }                                                                                         \
   __attribute__((constructor)) static void REF_CAT(REF_CAT(regu, NAME), SDXTYPE)(void)      \
   {  ref_un_table[ID][REF_IDX] = REF_CAT(REF_CAT(refu, NAME), SDXTYPE); }

REF_UN(fabs, RU_FABS, SOLID_OP_FABS, SDXTYPE)
REF_UN(sign, RU_SIGN, SOLID_OP_SIGN, SDXTYPE)
#if (!SDTYPE_IS_UNSIGNED_INT(SDXTYPE) && !SDTYPE_IS_BOOL(SDXTYPE))
REF_UN(negative, RU_NEGATIVE, SOLID_OP_NEGATIVE, SDXTYPE)
#endif
#if (SDTYPE_IS_BOOL(SDXTYPE))
REF_UN(lnot, RU_LNOT, SOLID_OP_BITNOT, SDXTYPE)
REF_UN(negative, RU_NEGATIVE, SOLID_OP_BITNOT, SDXTYPE)
#endif
#if (SDTYPE_IS_INT(SDXTYPE) || SDTYPE_IS_BOOL(SDXTYPE))
REF_UN(bitnot, RU_BITNOT, SOLID_OP_BITNOT, SDXTYPE)
#endif
#if (SDTYPE_IS_COMPLEX(SDXTYPE))
REF_UN(conj, RU_CONJ, SOLID_OP_CONJ, SDXTYPE)
REF_UN(absolute, RU_ABSOLUTE, SOLID_OP_ABSOLUTE, SDTYPE_ELEMTYPE(SDXTYPE))
#else
REF_UN(absolute, RU_ABSOLUTE, SOLID_OP_FABS, SDXTYPE)
#endif
#if (SDTYPE_IS_FLOAT(SDXTYPE) || SDTYPE_IS_COMPLEX(SDXTYPE))
REF_UN(ceil, RU_CEIL, SOLID_OP_CEIL, SDXTYPE)
REF_UN(floor, RU_FLOOR, SOLID_OP_FLOOR, SDXTYPE)
REF_UN(trunc, RU_TRUNC, SOLID_OP_TRUNC, SDXTYPE)
REF_UN(round, RU_ROUND, SOLID_OP_ROUND, SDXTYPE)
#endif
#if (!SDTYPE_IS_BOOL(SDXTYPE))
REF_UN(sin, RU_SIN, SOLID_OP_SIN, SDXTYPE)          REF_UN(cos, RU_COS, SOLID_OP_COS, SDXTYPE)
REF_UN(tan, RU_TAN, SOLID_OP_TAN, SDXTYPE)          REF_UN(sinh, RU_SINH, SOLID_OP_SINH, SDXTYPE)
REF_UN(cosh, RU_COSH, SOLID_OP_COSH, SDXTYPE)       REF_UN(tanh, RU_TANH, SOLID_OP_TANH, SDXTYPE)
REF_UN(arcsin, RU_ARCSIN, SOLID_OP_ARCSIN, SDXTYPE) REF_UN(arccos, RU_ARCCOS, SOLID_OP_ARCCOS, SDXTYPE)
REF_UN(arctan, RU_ARCTAN, SOLID_OP_ARCTAN, SDXTYPE) REF_UN(arcsinh, RU_ARCSINH, SOLID_OP_ARCSINH, SDXTYPE)
REF_UN(arccosh, RU_ARCCOSH, SOLID_OP_ARCCOSH, SDXTYPE) REF_UN(arctanh, RU_ARCTANH, SOLID_OP_ARCTANH, SDXTYPE)
REF_UN(reciprocal, RU_RECIPROCAL, SOLID_OP_RECIPROCAL, SDXTYPE)
REF_UN(sqrt, RU_SQRT, SOLID_OP_SQRT_312, SDXTYPE)   REF_UN(cbrt, RU_CBRT, SOLID_OP_CBRT, SDXTYPE)
REF_UN(square, RU_SQUARE, SOLID_OP_SQUARE, SDXTYPE) REF_UN(exp, RU_EXP, SOLID_OP_EXP, SDXTYPE)
REF_UN(exp2, RU_EXP2, SOLID_OP_EXP2, SDXTYPE)       REF_UN(exp10, RU_EXP10, SOLID_OP_EXP10, SDXTYPE)
REF_UN(expm1, RU_EXPM1, SOLID_OP_EXPM1, SDXTYPE)    REF_UN(log, RU_LOG, SOLID_OP_LOG, SDXTYPE)
REF_UN(log2, RU_LOG2, SOLID_OP_LOG2, SDXTYPE)       REF_UN(log10, RU_LOG10, SOLID_OP_LOG10, SDXTYPE)
REF_UN(log1p, RU_LOG1P, SOLID_OP_LOG1P, SDXTYPE)
#endif
REF_UN(isinf, RU_ISINF, SOLID_OP_ISINF, bool)
REF_UN(isnan, RU_ISNAN, SOLID_OP_ISNAN, bool)
REF_UN(isfinite, RU_ISFINITE, SOLID_OP_ISFINITE, bool)
#if (!SDTYPE_IS_COMPLEX(SDXTYPE))
REF_UN(isposinf, RU_ISPOSINF, SOLID_OP_ISPOSINF, bool)
REF_UN(isneginf, RU_ISNEGINF, SOLID_OP_ISNEGINF, bool)
#endif

/* ---- reductions: serial fold of a contiguous vector with the reference's
   init / accumulate / finalize code (reduce_ops.h); `prm` points to the op's parameter
   struct (bounds in the work type, or phalf/pinv for norm) ---- */
#include "solid/core/generic/reduce_ops.h"
#ifndef SOLID_OP_REDUCE_BREAK
#define SOLID_OP_REDUCE_BREAK  { _index = _n; break; }
#endif
#define REF_PARAM_0(NAME, PARAM)
#define REF_PARAM_1(NAME, PARAM) typedef struct PARAM REF_CAT(REF_CAT(refp, NAME), SDXTYPE);
#define REF_PARAMUSE_0(NAME)
#define REF_PARAMUSE_1(NAME) REF_CAT(REF_CAT(refp, NAME), SDXTYPE) param = *(const REF_CAT(REF_CAT(refp, NAME), SDXTYPE) *)prm;
#define REF_FINAL_0(RTYPE, CODE)
#define REF_FINAL_1(RTYPE, CODE) { SOLID_C_WORKTYPE_TYPE(RTYPE) _temp = _accumulate; SOLID_C_WORKTYPE_TYPE(RTYPE) *_partial = &_temp; \
                                   SOLID_C_WORKTYPE_TYPE(RTYPE) *_result = &_accumulate; CODE }
#define REF_SEL_(P, F) P##F
#define REF_SEL(P, F) REF_SEL_(P, F)
#define SD_TEMPLATE_REDUCE(NAME, DTYPE1, DTYPE2, FLAG_PARAM, PARAM, FLAG_INIT, FLAG_FINALIZE, \
                           CODE_INIT, CODE_ACCUMULATE, CODE_REDUCE, CODE_FINALIZE)           \
   REF_SEL(REF_PARAM_, FLAG_PARAM)(NAME, PARAM)                                              \
   static void REF_CAT(REF_CAT(refr, NAME), SDXTYPE)(size_t _n, const void *x, const void *prm, void *result) \
   {  SOLID_C_TYPE(DTYPE1) *_ptr = (SOLID_C_TYPE(DTYPE1) *)x;                                \
      SOLID_C_WORKTYPE_TYPE(DTYPE2) _accumulate; size_t _index;                              \
      REF_SEL(REF_PARAMUSE_, FLAG_PARAM)(NAME)                                               \
      CODE_INIT                                                                              \
      for (_index = 0; _index < _n; _index++) { CODE_ACCUMULATE _ptr++; }                    \
      REF_SEL(REF_FINAL_, FLAG_FINALIZE)(DTYPE2, CODE_FINALIZE)                              \
      SOLID_ASSIGN(SOLID_WORKTYPE(DTYPE2), DTYPE2, &_accumulate, result)                     \
      (void)prm;                                                                             \
   }
#define REF_RED(NAME, ID, MACRO)                                                             \
   MACRO                                                                                     \
   __attribute__((constructor)) static void REF_CAT(REF_CAT(regr, NAME), SDXTYPE)(void)      \
   {  ref_red_table[ID][REF_IDX] = REF_CAT(REF_CAT(refr, NAME), SDXTYPE); }

REF_RED(any, RR_ANY, SOLID_OP_REDUCE_ANY)
REF_RED(all, RR_ALL, SOLID_OP_REDUCE_ALL)
REF_RED(nnz, RR_NNZ, SOLID_OP_REDUCE_NNZ)
REF_RED(all_lt, RR_ALL_LT, SOLID_OP_REDUCE_ALL_LT)
REF_RED(all_le, RR_ALL_LE, SOLID_OP_REDUCE_ALL_LE)
REF_RED(all_gt, RR_ALL_GT, SOLID_OP_REDUCE_ALL_GT)
REF_RED(all_ge, RR_ALL_GE, SOLID_OP_REDUCE_ALL_GE)
REF_RED(all_gtlt, RR_ALL_GTLT, SOLID_OP_REDUCE_ALL_GTLT)
REF_RED(all_gtle, RR_ALL_GTLE, SOLID_OP_REDUCE_ALL_GTLE)
REF_RED(all_gelt, RR_ALL_GELT, SOLID_OP_REDUCE_ALL_GELT)
REF_RED(all_gele, RR_ALL_GELE, SOLID_OP_REDUCE_ALL_GELE)
REF_RED(sum, RR_SUM, SOLID_OP_REDUCE_SUM)
REF_RED(prod, RR_PROD, SOLID_OP_REDUCE_PROD)
REF_RED(sum_nan, RR_SUM_NAN, SOLID_OP_REDUCE_SUM_NAN)
REF_RED(prod_nan, RR_PROD_NAN, SOLID_OP_REDUCE_PROD_NAN)
REF_RED(sum_abs, RR_SUM_ABS, SOLID_OP_REDUCE_SUM_ABS)
REF_RED(sum_abs_nan, RR_SUM_ABS_NAN, SOLID_OP_REDUCE_SUM_ABS_NAN)
REF_RED(maximum, RR_MAXIMUM, SOLID_OP_REDUCE_MAXIMUM)
REF_RED(minimum, RR_MINIMUM, SOLID_OP_REDUCE_MINIMUM)
REF_RED(maximum_abs, RR_MAXIMUM_ABS, SOLID_OP_REDUCE_MAXIMUM_ABS)
REF_RED(minimum_abs, RR_MINIMUM_ABS, SOLID_OP_REDUCE_MINIMUM_ABS)
REF_RED(norm, RR_NORM, SOLID_OP_REDUCE_NORM)
REF_RED(norm2, RR_NORM2, SOLID_OP_REDUCE_NORM2)
#if (SDTYPE_IS_FLOAT(SDXTYPE) || SDTYPE_IS_COMPLEX(SDXTYPE))
REF_RED(all_finite, RR_ALL_FINITE, SOLID_OP_REDUCE_ALL_FINITE)
REF_RED(any_inf, RR_ANY_INF, SOLID_OP_REDUCE_ANY_INF)
REF_RED(any_nan, RR_ANY_NAN, SOLID_OP_REDUCE_ANY_NAN)
REF_RED(nnz_nan, RR_NNZ_NAN, SOLID_OP_REDUCE_NNZ_NAN)
REF_RED(norm_nan, RR_NORM_NAN, SOLID_OP_REDUCE_NORM_NAN)
REF_RED(norm2_nan, RR_NORM2_NAN, SOLID_OP_REDUCE_NORM2_NAN)
#endif

#undef SD_TEMPLATE_REDUCE
#undef REF_T
#undef REF_IDX
#endif
