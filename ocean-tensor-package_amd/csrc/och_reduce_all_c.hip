/* Full-reduction kernels, operations 15..20 of the reduction list. */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_c(int op, int dtype)
{
   switch (op)
   {
      case 15: return RowR<15>::fn[dtype];
      case 16: return RowR<16>::fn[dtype];
      case 17: return RowR<17>::fn[dtype];
      case 18: return RowR<18>::fn[dtype];
      case 19: return RowR<19>::fn[dtype];
      case 20: return RowR<20>::fn[dtype];
   }
   return nullptr;
}
}
