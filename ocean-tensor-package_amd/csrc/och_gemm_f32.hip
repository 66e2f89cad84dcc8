/* float GEMM: block tiles of 128 x 128 (64 x 64 per wave, 2 x 2 tiles of 32x32x2), 128 x 64, 64 x 128 or 64 x 64, K slab 16;
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 106 / 100 / 97 / 91 TFLOP/s. */
#include "och_gemm.h"
namespace och {
int gemm_float(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   switch (gemm_pick_tile(g, choice, 4))
   {  case 0:  return launch_gemm_mfma<float, false, 64, 64, 16>(g);
      case 1:  return launch_gemm_mfma<float, false, 64, 32, 16>(g);
      case 2:  return launch_gemm_mfma<float, false, 32, 64, 16>(g);
      default: return launch_gemm_mfma<float, false, 32, 32, 16>(g);
   }
}
}
