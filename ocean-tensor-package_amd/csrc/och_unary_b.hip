/* Unary elementwise kernels, operations 11..19 of the unary operation list. */
#include "och_unary_tmpl.h"
namespace och {
ew2_fn unary_lookup_b(int op, int dtype)
{
   switch (op)
   {
      case 11: return RowU<11>::fn[dtype];
      case 12: return RowU<12>::fn[dtype];
      case 13: return RowU<13>::fn[dtype];
      case 14: return RowU<14>::fn[dtype];
      case 15: return RowU<15>::fn[dtype];
      case 16: return RowU<16>::fn[dtype];
      case 17: return RowU<17>::fn[dtype];
      case 18: return RowU<18>::fn[dtype];
      case 19: return RowU<19>::fn[dtype];
   }
   return nullptr;
}
}
