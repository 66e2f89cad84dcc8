/* Axis-reduction kernels, operations: 3 4 5 6 */
#include "och_reduce_axis.h"
namespace och {
axis_fn axis_lookup_b(int op, int dtype)
{
   switch (op)
   {
      case 3: return RowA<3>::fn[dtype];
      case 4: return RowA<4>::fn[dtype];
      case 5: return RowA<5>::fn[dtype];
      case 6: return RowA<6>::fn[dtype];
   }
   return nullptr;
}
}
