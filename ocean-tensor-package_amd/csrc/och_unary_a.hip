/* Unary elementwise kernels, operations 0..10 of the unary operation list. */
#include "och_unary_tmpl.h"
namespace och {
ew2_fn unary_lookup_a(int op, int dtype)
{
   switch (op)
   {
      case 0: return RowU<0>::fn[dtype];
      case 1: return RowU<1>::fn[dtype];
      case 2: return RowU<2>::fn[dtype];
      case 3: return RowU<3>::fn[dtype];
      case 4: return RowU<4>::fn[dtype];
      case 5: return RowU<5>::fn[dtype];
      case 6: return RowU<6>::fn[dtype];
      case 7: return RowU<7>::fn[dtype];
      case 8: return RowU<8>::fn[dtype];
      case 9: return RowU<9>::fn[dtype];
      case 10: return RowU<10>::fn[dtype];
   }
   return nullptr;
}
}
