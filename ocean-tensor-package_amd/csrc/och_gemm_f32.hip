/* float GEMM: block tiles of 128 x 128 (64 x 64 per wave, 2 x 2 tiles of 32x32x2), 128 x 64, 64 x 128 or 64 x 64, K slab 16;
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 106 / 100 / 97 / 91 TFLOP/s. */
#include "och_gemm.h"
namespace och {
int gemm_float(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   const int pick = gemm_pick_tile(g, choice, 4);
   /* Aligned products with M and N multiples of 4 and K of 32 run on the pipelined kernel (och_gemm_f32p.hip) on tiles of
      256 x 256 or 128 x 128 when that is cheaper by the model of gemm_pick_tile: rounds of the compute units x tile area /
      efficiency, with the kernels below at 0.8 of the pipelined kernel on 256 x 256 tiles and the 128 x 128 tiles at 0.95
      (8192^3: 130 against 153 TFLOP/s; 2048^3: 84 against 135). A K that is not a multiple of 32 (scalars in host memory
      only): the whole slabs there, the rest of K as a product of its own that adds to C. */
   if (g.M >= 128 && g.N >= 128 && g.M % 4 == 0 && g.N % 4 == 0 && g.K >= 32 && (g.K % 32 == 0 || (g.scalar_mode_host && g.K >= 256)) && gemm_operands_aligned(g, 4))
   {  const uint64_t units = (uint64_t)gemm_compute_units();
      auto cost = [&](uint64_t bm, uint64_t bn, double efficiency)
      {  const uint64_t tiles = ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * (uint64_t)g.nz;
         return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
      };
      /* the pipelined kernel cuts the tiles of a last round that is at most half full along K: that round then counts as
         1 / shares of a round */
      GemmArgs whole = g;
      whole.K = g.K - g.K % 32;
      double rounds_large = 0, rounds_small = 0;
      gemm_float_pipe_split(whole, 256, &rounds_large); gemm_float_pipe_split(whole, 128, &rounds_small);
      /* what a block spends outside its main loop, in slabs of 32 k: about three on the large tile and in the kernels
         below, two on the small tile (8192 x 8192 x 256: 109, 93 and 118 TFLOP/s) */
      const double slabs = (double)(whole.K / 32);
      const double large = rounds_large * 65536.0 * (slabs + 3) / slabs, small = rounds_small * 16384.0 / 0.95 * (slabs + 2) / slabs;
      const double others = cost(choice[pick].bm, choice[pick].bn, choice[pick].efficiency * 0.8) * (slabs + 3) / slabs;
      const int forced = gemm_kernel_choice();
      const int tile = forced == 1 ? 256 : (forced == 2 ? 128 : (large <= small ? 256 : 128));
      if (forced != 3 && (forced != 0 || (tile == 256 ? large : small) < others))
      {  static const float one = 1.0f;
         const int done = gemm_pipelined_head_and_rest(g, 32, 4, &one, [&](const GemmArgs &a) { return gemm_float_pipe(a, tile); }, gemm_float);
         if (done <= 0) return done;
      }
   }
   switch (pick)
   {  case 0:  return launch_gemm_mfma<float, false, 64, 64, 16>(g);
      case 1:  return launch_gemm_mfma<float, false, 64, 32, 16>(g);
      case 2:  return launch_gemm_mfma<float, false, 32, 64, 16>(g);
      default: return launch_gemm_mfma<float, false, 32, 32, 16>(g);
   }
}
}
