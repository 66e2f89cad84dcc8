/* Axis-reduction kernels, operations: 15 16 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_c(int op, int dtype)
{
   switch (op)
   {
      case 15: return RowA<15>::fn[dtype];
      case 16: return RowA<16>::fn[dtype];
   }
   return nullptr;
}
}
