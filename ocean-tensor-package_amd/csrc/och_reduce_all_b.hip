/* Full-reduction kernels, operations: 4 5 6 7 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_b(int op, int dtype)
{
   switch (op)
   {
      case 4: return RowR<4>::fn[dtype];
      case 5: return RowR<5>::fn[dtype];
      case 6: return RowR<6>::fn[dtype];
      case 7: return RowR<7>::fn[dtype];
   }
   return nullptr;
}
}
