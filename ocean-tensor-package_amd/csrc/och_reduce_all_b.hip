/* Full-reduction kernels, operations 8..14 of the reduction list. */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_b(int op, int dtype)
{
   switch (op)
   {
      case 8: return RowR<8>::fn[dtype];
      case 9: return RowR<9>::fn[dtype];
      case 10: return RowR<10>::fn[dtype];
      case 11: return RowR<11>::fn[dtype];
      case 12: return RowR<12>::fn[dtype];
      case 13: return RowR<13>::fn[dtype];
      case 14: return RowR<14>::fn[dtype];
   }
   return nullptr;
}
}
