/* Binary elementwise kernels, part 2: power, remainders, pairwise minimum / maximum. */
#include "och_dispatch.h"
#include "och_ops_binary.h"
namespace och {
ew3_fn binary_lookup_misc(int op, int dtype)
{
   switch (op)
   {  case OCH_POWER: return Row3<BinPower, TS_ALL>::fn[dtype];
      case OCH_MOD:   return Row3<BinMod, TS_NOT_COMPLEX>::fn[dtype];
      case OCH_FMOD:  return Row3<BinFMod, TS_NOT_COMPLEX>::fn[dtype];
      case OCH_MIN:   return Row3<BinMin, TS_ALL>::fn[dtype];
      case OCH_MAX:   return Row3<BinMax, TS_ALL>::fn[dtype];
      case OCH_FMIN:  return Row3<BinFMin, TS_ALL>::fn[dtype];
      case OCH_FMAX:  return Row3<BinFMax, TS_ALL>::fn[dtype];
   }
   return nullptr;
}
}
