/* Axis-reduction kernels, operations: 25 26 27 28 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_d(int op, int dtype)
{
   switch (op)
   {
      case 25: return RowA<25>::fn[dtype];
      case 26: return RowA<26>::fn[dtype];
      case 27: return RowA<27>::fn[dtype];
      case 28: return RowA<28>::fn[dtype];
   }
   return nullptr;
}
}
