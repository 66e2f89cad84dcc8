/* cdouble GEMM: 128 x 64 block tile, 64 x 32 per wave, real and imaginary planes, K slab 8 */
#include "och_gemm.h"
namespace och { int gemm_cdouble(const GemmArgs &g) { return launch_gemm_mfma<double, true, 64, 32, 8>(g); } }
