/* Full-reduction kernels, operations: 12 13 14 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_d(int op, int dtype)
{
   switch (op)
   {
      case 12: return RowR<12>::fn[dtype];
      case 13: return RowR<13>::fn[dtype];
      case 14: return RowR<14>::fn[dtype];
   }
   return nullptr;
}
}
