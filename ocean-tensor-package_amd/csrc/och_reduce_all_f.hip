/* Full-reduction kernels, operations: 19 20 21 22 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_f(int op, int dtype)
{
   switch (op)
   {
      case 19: return RowR<19>::fn[dtype];
      case 20: return RowR<20>::fn[dtype];
      case 21: return RowR<21>::fn[dtype];
      case 22: return RowR<22>::fn[dtype];
   }
   return nullptr;
}
}
