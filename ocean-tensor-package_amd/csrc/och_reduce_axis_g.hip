/* Axis-reduction kernels, operations: 25 26 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_g(int op, int dtype)
{
   switch (op)
   {
      case 25: return RowA<25>::fn[dtype];
      case 26: return RowA<26>::fn[dtype];
   }
   return nullptr;
}
}
