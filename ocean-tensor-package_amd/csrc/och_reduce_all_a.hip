/* Full-reduction kernels, operations 0..7 of the reduction list. */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_a(int op, int dtype)
{
   switch (op)
   {
      case 0: return RowR<0>::fn[dtype];
      case 1: return RowR<1>::fn[dtype];
      case 2: return RowR<2>::fn[dtype];
      case 3: return RowR<3>::fn[dtype];
      case 4: return RowR<4>::fn[dtype];
      case 5: return RowR<5>::fn[dtype];
      case 6: return RowR<6>::fn[dtype];
      case 7: return RowR<7>::fn[dtype];
   }
   return nullptr;
}
}
