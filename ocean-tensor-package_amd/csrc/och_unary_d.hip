/* Unary elementwise kernels, operations 29..39 of the unary operation list. */
#include "och_unary_tmpl.h"
namespace och {
ew2_fn unary_lookup_d(int op, int dtype)
{
   switch (op)
   {
      case 29: return RowU<29>::fn[dtype];
      case 30: return RowU<30>::fn[dtype];
      case 31: return RowU<31>::fn[dtype];
      case 32: return RowU<32>::fn[dtype];
      case 33: return RowU<33>::fn[dtype];
      case 34: return RowU<34>::fn[dtype];
      case 35: return RowU<35>::fn[dtype];
      case 36: return RowU<36>::fn[dtype];
      case 37: return RowU<37>::fn[dtype];
      case 38: return RowU<38>::fn[dtype];
      case 39: return RowU<39>::fn[dtype];
   }
   return nullptr;
}
}
