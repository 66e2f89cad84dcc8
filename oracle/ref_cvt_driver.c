/* TEST INFRASTRUCTURE -- second part of oracle/_ref: the reference's conversion macros
 * SOLID_ASSIGN and SOLID_BYTESWAP_ASSIGN (solid/include/solid/base/generic/dtype_assign.h)
 * instantiated for all 15 x 15 type pairs through the reference's generate_all_types2.h,
 * and SOLID_BYTESWAP for each type. See ref_ops_driver.c for why only the macro headers
 * (and not the CPU kernel sources) can be built here.
 */
#ifndef SD_TEMPLATE_FILE
#define SD_TEMPLATE_FILE "ref_cvt_driver.c"

#include <stddef.h>
#include <stdint.h>
#include "solid/base/generic/dtype_macros.h"
#include "solid/base/generic/dtype_assign.h"
#include "solid/base/cpu/dtype_cpu.h"

#define REFC_CAT3_(a, b, c) a##_##b##_##c
#define REFC_CAT3(a, b, c) REFC_CAT3_(a, b, c)

typedef void (*ref_cvt_fn)(size_t n, const void *x, void *y);
static ref_cvt_fn ref_assign_table[15][15];
static ref_cvt_fn ref_swap_assign_table[15][15];

ref_cvt_fn ref_assign(int ts, int td)      { return (ts >= 0 && ts < 15 && td >= 0 && td < 15) ? ref_assign_table[ts][td] : 0; }
ref_cvt_fn ref_swap_assign(int ts, int td) { return (ts >= 0 && ts < 15 && td >= 0 && td < 15) ? ref_swap_assign_table[ts][td] : 0; }

#include "solid/base/generic/generate_all_types2.h"

#else  /* SDXTYPE (source) and SDXTYPE2 (destination) are defined */

static void REFC_CAT3(refc_assign, SDXTYPE, SDXTYPE2)(size_t n, const void *x, void *y)
{  SOLID_C_TYPE(SDXTYPE) *px = (SOLID_C_TYPE(SDXTYPE) *)x; SOLID_C_TYPE(SDXTYPE2) *py = (SOLID_C_TYPE(SDXTYPE2) *)y; size_t i;
   for (i = 0; i < n; i++) { SOLID_ASSIGN(SDXTYPE, SDXTYPE2, px + i, py + i) }
}
static void REFC_CAT3(refc_swap, SDXTYPE, SDXTYPE2)(size_t n, const void *x, void *y)
{  SOLID_C_TYPE(SDXTYPE) *px = (SOLID_C_TYPE(SDXTYPE) *)x; SOLID_C_TYPE(SDXTYPE2) *py = (SOLID_C_TYPE(SDXTYPE2) *)y; size_t i;
   for (i = 0; i < n; i++) { SOLID_BYTESWAP_ASSIGN(SDXTYPE, SDXTYPE2, px + i, py + i) }
}
__attribute__((constructor)) static void REFC_CAT3(refc_reg, SDXTYPE, SDXTYPE2)(void)
{  ref_assign_table[SDTYPE_INDEX(SDXTYPE)][SDTYPE_INDEX(SDXTYPE2)] = REFC_CAT3(refc_assign, SDXTYPE, SDXTYPE2);
   ref_swap_assign_table[SDTYPE_INDEX(SDXTYPE)][SDTYPE_INDEX(SDXTYPE2)] = REFC_CAT3(refc_swap, SDXTYPE, SDXTYPE2);
}
#endif
