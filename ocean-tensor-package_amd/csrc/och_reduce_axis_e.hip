/* Axis-reduction kernels, operations: 19 20 21 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_e(int op, int dtype)
{
   switch (op)
   {
      case 19: return RowA<19>::fn[dtype];
      case 20: return RowA<20>::fn[dtype];
      case 21: return RowA<21>::fn[dtype];
   }
   return nullptr;
}
}
