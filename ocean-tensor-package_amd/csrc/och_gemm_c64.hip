/* cdouble GEMM: block tiles of 128 x 64 (64 x 32 per wave) or 64 x 64, K slab 8; chosen by gemm_pick_tile. */
#include "och_gemm.h"
namespace och {
int gemm_cdouble(const GemmArgs &g)
{  static const GemmTileChoice choice[2] = { { 128, 64, 1.0 }, { 64, 64, 0.94 } };
   const int pick = gemm_pick_tile(g, choice, 2);
   /* Products with K a multiple of 16 run on the pipelined kernel (och_gemm_c64p.hip) on tiles of 128 x 64 when that is
      cheaper by the model of gemm_pick_tile (rounds of the compute units x tile area / efficiency, the kernel below at
      0.87 of the pipelined one). A K that is not a multiple of 16 (scalars in host memory only): the whole slabs there,
      the rest of K as a product of its own that adds to C. */
   if (g.M >= 64 && g.N >= 32 && g.K >= 16 && (g.K % 16 == 0 || (g.scalar_mode_host && g.K >= 128)) && gemm_operands_aligned(g, 16))
   {  const uint64_t units = (uint64_t)gemm_compute_units();
      auto cost = [&](uint64_t bm, uint64_t bn, double efficiency)
      {  const uint64_t tiles = ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * (uint64_t)g.nz;
         return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
      };
      /* the pipelined kernel cuts the tiles of a last round that is at most half full along K: that round then counts as
         a fraction of a round */
      GemmArgs whole = g;
      whole.K = g.K - g.K % 16;
      double rounds = 0;
      gemm_cdouble_pipe_split(whole, &rounds);
      const double pipelined = rounds * 8192.0;
      const int forced = gemm_kernel_choice();
      if (forced != 3 && (forced != 0 || pipelined < cost(choice[pick].bm, choice[pick].bn, choice[pick].efficiency * 0.87)))
      {  static const double one[2] = { 1.0, 0.0 };
         const int done = gemm_pipelined_head_and_rest(g, 16, 16, one, [&](const GemmArgs &a) { return gemm_cdouble_pipe(a); }, gemm_cdouble);
         if (done <= 0) return done;
      }
   }
   if (pick == 0) return launch_gemm_mfma<double, true, 64, 32, 8>(g);
   return launch_gemm_mfma<double, true, 32, 32, 8>(g);
}
}
