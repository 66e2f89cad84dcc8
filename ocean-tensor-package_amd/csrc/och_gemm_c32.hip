/* cfloat GEMM: as float, with real and imaginary planes (four real MFMAs per tile), K slab 8. */
#include "och_gemm.h"
namespace och {
int gemm_cfloat(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   const int pick = gemm_pick_tile(g, choice, 4);
   /* Aligned products with M and N multiples of 2 and K of 32 run on the pipelined kernel on tiles of 128 x 128 when
      that is cheaper by the model of gemm_pick_tile (rounds of the compute units x tile area / efficiency, the kernels
      below at 0.87 of the pipelined one). A K that is not a multiple of 32 (scalars in host memory only): the whole
      slabs there, the rest of K as a product of its own that adds to C. */
   if (g.M >= 128 / 2 && g.N >= 128 / 2 && g.M % 2 == 0 && g.N % 2 == 0 && g.K >= 32 && (g.K % 32 == 0 || (g.scalar_mode_host && g.K >= 256)) && gemm_operands_aligned(g, 8))
   {  const uint64_t units = (uint64_t)gemm_compute_units();
      auto cost = [&](uint64_t bm, uint64_t bn, double efficiency)
      {  const uint64_t tiles = ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * (uint64_t)g.nz;
         return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
      };
      /* the pipelined kernel cuts the tiles of a last round that is at most half full along K: that round then counts as
         a fraction of a round */
      GemmArgs whole = g;
      whole.K = g.K - g.K % 32;
      double rounds = 0;
      gemm_cfloat_pipe_split(whole, &rounds);
      const double pipelined = rounds * 16384.0;
      const int forced = gemm_kernel_choice();
      if (forced != 3 && (forced != 0 || pipelined < cost(choice[pick].bm, choice[pick].bn, choice[pick].efficiency * 0.87)))
      {  static const float one[2] = { 1.0f, 0.0f };
         const int done = gemm_pipelined_head_and_rest(g, 32, 8, one, [&](const GemmArgs &a) { return gemm_cfloat_pipe(a); }, gemm_cfloat);
         if (done <= 0) return done;
      }
   }
   switch (pick)
   {  case 0:
         return launch_gemm_mfma<float, true, 64, 64, 8>(g);
      case 1:  return launch_gemm_mfma<float, true, 64, 32, 8>(g);
      case 2:  return launch_gemm_mfma<float, true, 32, 64, 8>(g);
      default: return launch_gemm_mfma<float, true, 32, 32, 8>(g);
   }
}
}
