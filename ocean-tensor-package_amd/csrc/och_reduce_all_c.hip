/* Full-reduction kernels, operations: 8 9 10 11 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_c(int op, int dtype)
{
   switch (op)
   {
      case 8: return RowR<8>::fn[dtype];
      case 9: return RowR<9>::fn[dtype];
      case 10: return RowR<10>::fn[dtype];
      case 11: return RowR<11>::fn[dtype];
   }
   return nullptr;
}
}
