/* double GEMM: 128 x 128 block tile, 64 x 64 per wave (4 x 4 tiles of 16x16x4), K slab 8 */
#include "och_gemm.h"
namespace och { int gemm_double(const GemmArgs &g) { return launch_gemm_mfma<double, false, 64, 64, 8>(g); } }
