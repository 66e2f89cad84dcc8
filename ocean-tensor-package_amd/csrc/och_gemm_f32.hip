/* float GEMM: 128 x 128 block tile, 64 x 64 per wave (2 x 2 tiles of 32x32x2), K slab 16.
   Products with too few of those tiles to occupy the device use 64 x 64 block tiles instead. */
#include "och_gemm.h"
namespace och {
int gemm_float(const GemmArgs &g)
{  if (gemm_few_tiles(g, 128, 128)) return launch_gemm_mfma<float, false, 32, 32, 16>(g);
   return launch_gemm_mfma<float, false, 64, 64, 16>(g);
}
}
