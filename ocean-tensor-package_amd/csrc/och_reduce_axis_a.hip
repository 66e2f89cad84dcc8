/* Axis-reduction kernels, operations: 0 1 2 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_a(int op, int dtype)
{
   switch (op)
   {
      case 0: return RowA<0>::fn[dtype];
      case 1: return RowA<1>::fn[dtype];
      case 2: return RowA<2>::fn[dtype];
   }
   return nullptr;
}
}
