/* Unary elementwise kernels, operations 20..28 of the unary operation list. */
#include "och_unary_tmpl.h"
namespace och {
ew2_fn unary_lookup_c(int op, int dtype)
{
   switch (op)
   {
      case 20: return RowU<20>::fn[dtype];
      case 21: return RowU<21>::fn[dtype];
      case 22: return RowU<22>::fn[dtype];
      case 23: return RowU<23>::fn[dtype];
      case 24: return RowU<24>::fn[dtype];
      case 25: return RowU<25>::fn[dtype];
      case 26: return RowU<26>::fn[dtype];
      case 27: return RowU<27>::fn[dtype];
      case 28: return RowU<28>::fn[dtype];
   }
   return nullptr;
}
}
