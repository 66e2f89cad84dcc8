/* Full-reduction kernels, operations: 26 27 28 */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_h(int op, int dtype)
{
   switch (op)
   {
      case 26: return RowR<26>::fn[dtype];
      case 27: return RowR<27>::fn[dtype];
      case 28: return RowR<28>::fn[dtype];
   }
   return nullptr;
}
}
