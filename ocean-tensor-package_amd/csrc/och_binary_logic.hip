/* Binary elementwise kernels, part 3: comparisons, bitwise / logical operations, shifts. */
#include "och_dispatch.h"
#include "och_ops_binary.h"
namespace och {
ew3_fn binary_lookup_logic(int op, int dtype)
{
   switch (op)
   {  case OCH_LT: return Row3<BinLT, TS_ALL>::fn[dtype];
      case OCH_LE: return Row3<BinLE, TS_ALL>::fn[dtype];
      case OCH_EQ: return Row3<BinEQ, TS_ALL>::fn[dtype];
      case OCH_NE: return Row3<BinNE, TS_ALL>::fn[dtype];
      case OCH_GE: return Row3<BinGE, TS_ALL>::fn[dtype];
      case OCH_GT: return Row3<BinGT, TS_ALL>::fn[dtype];
      case OCH_BITWISE_AND: return Row3<BinBitAnd, TS_INT_BOOL>::fn[dtype];
      case OCH_BITWISE_OR:  return Row3<BinBitOr,  TS_INT_BOOL>::fn[dtype];
      case OCH_BITWISE_XOR: return Row3<BinBitXor, TS_INT_BOOL>::fn[dtype];
      case OCH_LOGICAL_AND: return Row3<BinBitAnd, TS_BOOL>::fn[dtype];
      case OCH_LOGICAL_OR:  return Row3<BinBitOr,  TS_BOOL>::fn[dtype];
      case OCH_LOGICAL_XOR: return Row3<BinBitXor, TS_BOOL>::fn[dtype];
      case OCH_BITSHIFT_LEFT:  return Row3<BinShiftLeft,  TS_INT_BOOL>::fn[dtype];
      case OCH_BITSHIFT_RIGHT: return Row3<BinShiftRight, TS_INT_BOOL>::fn[dtype];
   }
   return nullptr;
}
}
