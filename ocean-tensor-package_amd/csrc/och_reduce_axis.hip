/* C ABI of the axis reductions (och_reduce_axis). The 21 operations of the reference's axis
 * family (solid_core_gpu.src: axis_any ... axis_norm2_nan) are available; the range checks
 * (all_lt ...) exist as full reductions only. */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_a(int op, int dtype);
axis_fn axis_lookup_b(int op, int dtype);
axis_fn axis_lookup_c(int op, int dtype);
axis_fn axis_lookup_d(int op, int dtype);
}
extern "C" int och_reduce_axis(int op, int dtype, const och_reduce_axis_config *config, double p)
{
   using namespace och;
   axis_fn fn = nullptr;
   if (dtype >= 0 && dtype < DT_COUNT)
   {  if (op >= OCH_R_ANY && op <= OCH_R_NNZ_NAN) fn = axis_lookup_a(op, dtype);
      else if (op >= OCH_R_SUM && op <= OCH_R_PROD_NAN) fn = axis_lookup_b(op, dtype);
      else if (op >= OCH_R_SUM_ABS && op <= OCH_R_MINIMUM_ABS) fn = axis_lookup_c(op, dtype);
      else if (op >= OCH_R_NORM && op <= OCH_R_NORM2_NAN) fn = axis_lookup_d(op, dtype);
   }
   if (fn == nullptr) return set_error("axis reduction %d is not available for data type %d", op, dtype);
   return fn(config, p);
}
