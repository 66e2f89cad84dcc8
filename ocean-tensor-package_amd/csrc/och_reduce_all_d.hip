/* Full-reduction kernels, operations 21..28 of the reduction list. */
#include "och_reduce_all.h"
namespace och {
red_fn reduce_lookup_d(int op, int dtype)
{
   switch (op)
   {
      case 21: return RowR<21>::fn[dtype];
      case 22: return RowR<22>::fn[dtype];
      case 23: return RowR<23>::fn[dtype];
      case 24: return RowR<24>::fn[dtype];
      case 25: return RowR<25>::fn[dtype];
      case 26: return RowR<26>::fn[dtype];
      case 27: return RowR<27>::fn[dtype];
      case 28: return RowR<28>::fn[dtype];
   }
   return nullptr;
}
}
