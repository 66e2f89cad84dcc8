/* Axis-reduction kernels, operations: 22 23 24 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_f(int op, int dtype)
{
   switch (op)
   {
      case 22: return RowA<22>::fn[dtype];
      case 23: return RowA<23>::fn[dtype];
      case 24: return RowA<24>::fn[dtype];
   }
   return nullptr;
}
}
