/* double GEMM: block tiles of 128 x 128 (64 x 64 per wave, 4 x 4 tiles of 16x16x4), 128 x 64, 64 x 128 or 64 x 64, K slab 16 (two barriers fewer per 16 k than with slabs of 8: 8192^3 TN 64.3 -> 66.1, NT 66.3 -> 68.4 TFLOP/s);
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 56 / 55 / 55 / 53 TFLOP/s. */
#include "och_gemm.h"
namespace och {
int gemm_double(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.96 }, { 64, 128, 0.96 }, { 64, 64, 0.92 } };
   const int pick = gemm_pick_tile(g, choice, 4);
   /* Aligned products with M and N multiples of 2 and K of 16 run on the pipelined kernel on tiles of 256 x 128 or 128 x 128 (at 0.9) when
      that is cheaper by the model of gemm_pick_tile (rounds of the compute units x tile area / efficiency, the kernels
      below at 0.87 of the pipelined one). A K that is not a multiple of 16 (scalars in host memory only): the whole
      slabs there, the rest of K as a product of its own that adds to C. */
   if (g.M >= 256 / 2 && g.N >= 128 / 2 && g.M % 2 == 0 && g.N % 2 == 0 && g.K >= 16 && (g.K % 16 == 0 || (g.scalar_mode_host && g.K >= 128)) && gemm_operands_aligned(g, 8))
   {  const uint64_t units = (uint64_t)gemm_compute_units();
      auto cost = [&](uint64_t bm, uint64_t bn, double efficiency)
      {  const uint64_t tiles = ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * (uint64_t)g.nz;
         return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
      };
      /* the pipelined kernel cuts the tiles of a last round that is at most half full along K: that round then counts as
         1 / shares of a round */
      GemmArgs whole = g;
      whole.K = g.K - g.K % 16;
      double rounds_large = 0, rounds_small = 0;
      gemm_double_pipe_split(whole, 256, &rounds_large); gemm_double_pipe_split(whole, 128, &rounds_small);
      /* what a block spends outside its main loop, in slabs of 16 k: about three on the large tile, two on the small one,
         four in the kernels below */
      const double slabs = (double)(whole.K / 16);
      const double large = rounds_large * 32768.0 * (slabs + 3) / slabs, small = rounds_small * 16384.0 / 0.95 * (slabs + 2) / slabs;
      const int forced = gemm_kernel_choice();
      const int tile_m = forced == 1 ? 256 : (forced == 2 ? 128 : (large <= small ? 256 : 128));
      if (forced != 3 && (forced != 0 || (tile_m == 256 ? large : small) < cost(choice[pick].bm, choice[pick].bn, choice[pick].efficiency * 0.87) * (slabs + 4) / slabs))
      {  static const double one = 1.0;
         const int done = gemm_pipelined_head_and_rest(g, 16, 8, &one, [&](const GemmArgs &a) { return gemm_double_pipe(a, tile_m); }, gemm_double);
         if (done <= 0) return done;
      }
   }
   switch (pick)
   {  case 0:
         return launch_gemm_mfma<double, false, 64, 64, 16>(g);
      case 1:  return launch_gemm_mfma<double, false, 64, 32, 16>(g);
      case 2:  return launch_gemm_mfma<double, false, 32, 64, 16>(g);
      default: return launch_gemm_mfma<double, false, 32, 32, 16>(g);
   }
}
}
