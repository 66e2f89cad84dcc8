/* Axis-reduction kernels, operations: 17 18 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_d(int op, int dtype)
{
   switch (op)
   {
      case 17: return RowA<17>::fn[dtype];
      case 18: return RowA<18>::fn[dtype];
   }
   return nullptr;
}
}
