/* Full-reduction kernels, operations: 15 16 17 18 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_e(int op, int dtype)
{
   switch (op)
   {
      case 15: return RowR<15>::fn[dtype];
      case 16: return RowR<16>::fn[dtype];
      case 17: return RowR<17>::fn[dtype];
      case 18: return RowR<18>::fn[dtype];
   }
   return nullptr;
}
}
