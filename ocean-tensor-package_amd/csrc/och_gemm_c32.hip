/* cfloat GEMM: as float, with real and imaginary planes (four real MFMAs per tile), K slab 8. */
#include "och_gemm.h"
namespace och {
int gemm_cfloat(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   switch (gemm_pick_tile(g, choice, 4))
   {  case 0:  return launch_gemm_mfma<float, true, 64, 64, 8>(g);
      case 1:  return launch_gemm_mfma<float, true, 64, 32, 8>(g);
      case 2:  return launch_gemm_mfma<float, true, 32, 64, 8>(g);
      default: return launch_gemm_mfma<float, true, 32, 32, 8>(g);
   }
}
}
