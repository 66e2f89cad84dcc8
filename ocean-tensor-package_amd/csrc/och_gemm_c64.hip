/* cdouble GEMM: block tiles of 128 x 64 (64 x 32 per wave) or 64 x 64, K slab 8; chosen by gemm_pick_tile. */
#include "och_gemm.h"
namespace och {
int gemm_cdouble(const GemmArgs &g)
{  static const GemmTileChoice choice[2] = { { 128, 64, 1.0 }, { 64, 64, 0.94 } };
   if (gemm_pick_tile(g, choice, 2) == 0) return launch_gemm_mfma<double, true, 64, 32, 8>(g);
   return launch_gemm_mfma<double, true, 32, 32, 8>(g);
}
}
