/* C ABI of the binary elementwise operations (och_binary and its queries). */
#include "och_dispatch.h"
namespace och {
ew3_fn binary_lookup_arith(int op, int dtype);
ew3_fn binary_lookup_misc(int op, int dtype);
ew3_fn binary_lookup_logic(int op, int dtype);

static ew3_fn binary_lookup(int op, int dtype)
{
   if (!dtype_ok(dtype) || op < 0 || op >= OCH_BINARY_COUNT) return nullptr;
   if (op <= OCH_FLOOR_DIVIDE) return binary_lookup_arith(op, dtype);
   if (op <= OCH_FMAX) return binary_lookup_misc(op, dtype);
   return binary_lookup_logic(op, dtype);
}
}

extern "C" int och_binary_supported(int op, int dtype) { return och::binary_lookup(op, dtype) != nullptr; }

extern "C" int och_binary_operand2_dtype(int op, int dtype)
{
   if (!och_binary_supported(op, dtype)) return -1;
   if (op == OCH_BITSHIFT_LEFT || op == OCH_BITSHIFT_RIGHT) return OCH_INT8;
   if (op == OCH_POWER && dtype <= OCH_INT64) return OCH_INT16;
   return dtype;
}

extern "C" int och_binary_result_dtype(int op, int dtype)
{
   if (!och_binary_supported(op, dtype)) return -1;
   return (op >= OCH_LT && op <= OCH_GT) ? OCH_BOOL : dtype;
}

extern "C" int och_binary(int op, int dtype, int ndims, const size_t *size,
                          const ptrdiff_t *strides1, void *ptr1,
                          const ptrdiff_t *strides2, void *ptr2,
                          const ptrdiff_t *strides3, void *ptr3, och_stream stream)
{
   och::ew3_fn fn = och::binary_lookup(op, dtype);
   if (fn == nullptr) return och::set_error("binary operation %d is not available for data type %d", op, dtype);
   if (ptr3 == nullptr && strides3 == nullptr)
   {  if (och_binary_result_dtype(op, dtype) != dtype)
         return och::set_error("binary operation %d cannot be applied in place", op);
      ptr3 = ptr1; strides3 = strides1;
   }
   return fn(ndims, size, strides1, ptr1, strides2, ptr2, strides3, ptr3, och::as_stream(stream));
}
