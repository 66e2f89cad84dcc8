/* Full-reduction kernels, operations: 0 1 2 3 */
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
   }
   return nullptr;
}
}
