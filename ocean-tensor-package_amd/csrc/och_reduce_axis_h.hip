/* Axis-reduction kernels, operations: 27 28 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_h(int op, int dtype)
{
   switch (op)
   {
      case 27: return RowA<27>::fn[dtype];
      case 28: return RowA<28>::fn[dtype];
   }
   return nullptr;
}
}
