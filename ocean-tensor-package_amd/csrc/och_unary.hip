/* C ABI of the unary elementwise operations (och_unary and its queries). */
#include "och_dispatch.h"
#include "och_ops_unary.h"
namespace och {
ew2_fn unary_lookup_a(int op, int dtype);
ew2_fn unary_lookup_b(int op, int dtype);
ew2_fn unary_lookup_c(int op, int dtype);
ew2_fn unary_lookup_d(int op, int dtype);
static ew2_fn unary_lookup(int op, int dtype)
{
   if (!dtype_ok(dtype) || op < 0 || op >= OCH_UNARY_COUNT) return nullptr;
   if (op <= 10) return unary_lookup_a(op, dtype);
   if (op <= 19) return unary_lookup_b(op, dtype);
   if (op <= 28) return unary_lookup_c(op, dtype);
   return unary_lookup_d(op, dtype);
}
static_assert((int)U_COUNT == (int)OCH_UNARY_COUNT, "operation lists out of step");
static_assert((int)U_ISNEGINF == (int)OCH_ISNEGINF && (int)U_ABSOLUTE == (int)OCH_ABSOLUTE && (int)U_SQRT == (int)OCH_SQRT, "operation lists out of step");
}

extern "C" int och_unary_supported(int op, int dtype) { return och::unary_lookup(op, dtype) != nullptr; }

extern "C" int och_unary_result_dtype(int op, int dtype)
{
   if (!och_unary_supported(op, dtype)) return -1;
   if (op >= OCH_ISINF) return OCH_BOOL;
   if (op == OCH_ABSOLUTE && dtype >= OCH_CHALF) return dtype - 3;     /* complex -> its part type */
   return dtype;
}

extern "C" int och_unary(int op, int dtype, int ndims, const size_t *size,
                         const ptrdiff_t *strides1, void *ptr1,
                         const ptrdiff_t *strides2, void *ptr2, och_stream stream)
{
   och::ew2_fn fn = och::unary_lookup(op, dtype);
   if (fn == nullptr) return och::set_error("unary operation %d is not available for data type %d", op, dtype);
   if (ptr2 == nullptr && strides2 == nullptr)
   {  if (och_unary_result_dtype(op, dtype) != dtype)
         return och::set_error("unary operation %d cannot be applied in place", op);
      ptr2 = ptr1; strides2 = strides1;
   }
   return fn(ndims, size, strides1, ptr1, strides2, ptr2, och::as_stream(stream));
}
