/* double GEMM: 128 x 128 block tile, 64 x 64 per wave (4 x 4 tiles of 16x16x4), K slab 8.
   Products with too few of those tiles to occupy the device use 64 x 64 block tiles instead. */
#include "och_gemm.h"
namespace och {
int gemm_double(const GemmArgs &g)
{  if (gemm_few_tiles(g, 128, 128)) return launch_gemm_mfma<double, false, 32, 32, 8>(g);
   return launch_gemm_mfma<double, false, 64, 64, 8>(g);
}
}
