/* cdouble GEMM: 128 x 64 block tile, 64 x 32 per wave, real and imaginary planes, K slab 8.
   Products with too few of those tiles to occupy the device use 64 x 64 block tiles instead. */
#include "och_gemm.h"
namespace och {
int gemm_cdouble(const GemmArgs &g)
{  if (gemm_few_tiles(g, 128, 64)) return launch_gemm_mfma<double, true, 32, 32, 8>(g);
   return launch_gemm_mfma<double, true, 64, 32, 8>(g);
}
}
