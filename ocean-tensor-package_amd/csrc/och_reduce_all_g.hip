/* Full-reduction kernels, operations: 23 24 25 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_g(int op, int dtype)
{
   switch (op)
   {
      case 23: return RowR<23>::fn[dtype];
      case 24: return RowR<24>::fn[dtype];
      case 25: return RowR<25>::fn[dtype];
   }
   return nullptr;
}
}
