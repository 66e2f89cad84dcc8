/* double GEMM: block tiles of 128 x 128 (64 x 64 per wave, 4 x 4 tiles of 16x16x4), 128 x 64, 64 x 128 or 64 x 64, K slab 16 (two barriers fewer per 16 k than with slabs of 8: 8192^3 TN 64.3 -> 66.1, NT 66.3 -> 68.4 TFLOP/s);
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 56 / 55 / 55 / 53 TFLOP/s. */
#include "och_gemm.h"
namespace och {
int gemm_double(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.96 }, { 64, 128, 0.96 }, { 64, 64, 0.92 } };
   switch (gemm_pick_tile(g, choice, 4))
   {  case 0:  return launch_gemm_mfma<double, false, 64, 64, 16>(g);
      case 1:  return launch_gemm_mfma<double, false, 64, 32, 16>(g);
      case 2:  return launch_gemm_mfma<double, false, 32, 64, 16>(g);
      default: return launch_gemm_mfma<double, false, 32, 32, 16>(g);
   }
}
}
