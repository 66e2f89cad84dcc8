/* Binary elementwise kernels, part 1: add, subtract, multiply and the divisions. */
#include "och_dispatch.h"
#include "och_ops_binary.h"
namespace och {
ew3_fn binary_lookup_arith(int op, int dtype)
{
   switch (op)
   {  case OCH_ADD:          return Row3<BinAdd, TS_ALL>::fn[dtype];
      case OCH_SUBTRACT:     return Row3<BinSubtract, TS_ALL>::fn[dtype];
      case OCH_MULTIPLY:     return Row3<BinMultiply, TS_ALL>::fn[dtype];
      case OCH_DIVIDE:       return Row3<BinDivide, TS_ALL>::fn[dtype];
      case OCH_TRUE_DIVIDE:  return Row3<BinTrueDivide, TS_ALL>::fn[dtype];
      case OCH_FLOOR_DIVIDE: return Row3<BinFloorDivide, TS_NOT_COMPLEX>::fn[dtype];
   }
   return nullptr;
}
}
