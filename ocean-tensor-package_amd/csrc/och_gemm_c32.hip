/* cfloat GEMM: 128 x 128 block tile, 64 x 64 per wave, real and imaginary planes, K slab 8 */
#include "och_gemm.h"
namespace och { int gemm_cfloat(const GemmArgs &g) { return launch_gemm_mfma<float, true, 64, 64, 8>(g); } }
