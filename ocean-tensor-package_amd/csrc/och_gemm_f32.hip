/* float GEMM: block tiles of 128 x 128 (64 x 64 per wave, 2 x 2 tiles of 32x32x2), 128 x 64, 64 x 128 or 64 x 64, K slab 16;
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 106 / 100 / 97 / 91 TFLOP/s. */
#include "och_gemm.h"
namespace och {
int gemm_float(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   const int pick = gemm_pick_tile(g, choice, 4);
   /* Large aligned products with K a multiple of 32: the whole 256 x 256 or 128 x 128 tiles run on the pipelined kernel
      (och_gemm_f32p.hip), the strip of columns to their right and the strip of rows below them as products of their own --
      when that is cheaper by the model of gemm_pick_tile: rounds of the compute units x tile area / efficiency, with the
      kernels below at 0.85 of the pipelined kernel on 256 x 256 tiles and the 128 x 128 tiles at 0.9 (8192^3: 130 against
      153 TFLOP/s; 2048^3: 84 against 135). */
   if (g.M >= 128 && g.N >= 128 && g.K >= 32 && g.K % 32 == 0 && gemm_operands_aligned(g, 4))
   {  const uint64_t units = (uint64_t)gemm_compute_units();
      auto cost = [&](uint64_t bm, uint64_t bn, double efficiency, bool whole)
      {  const uint64_t tiles = (whole ? (g.M / bm) * (g.N / bn) : ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn)) * (uint64_t)g.nz;
         return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
      };
      const double others = cost(choice[pick].bm, choice[pick].bn, choice[pick].efficiency * 0.85, false);
      const double large = g.M >= 256 && g.N >= 256 ? cost(256, 256, 1.0, true) : 1e300, small = cost(128, 128, 0.9, true);
      const int tile = large <= small ? 256 : 128;
      if ((tile == 256 ? large : small) < others)
      {  const size_t Mi = g.M - g.M % tile, Ni = g.N - g.N % tile;
         GemmArgs part = g;
         part.M = Mi; part.N = Ni;
         const int taken = gemm_float_pipe(part, tile);
         if (taken < 0) return taken;
         if (taken == 0)
         {  if (g.N > Ni)
            {  part = g; part.N = g.N - Ni;
               part.B = (const char *)g.B + (int64_t)Ni * (g.transB == 'N' ? (int64_t)g.ldB : 1) * 4;
               part.C = (char *)g.C + (int64_t)Ni * g.ldC * 4;
               if (gemm_float(part) != 0) return -1;
            }
            if (g.M > Mi)
            {  part = g; part.M = g.M - Mi; part.N = Ni;
               part.A = (const char *)g.A + (int64_t)Mi * (g.transA == 'N' ? 1 : (int64_t)g.ldA) * 4;
               part.C = (char *)g.C + (int64_t)Mi * 4;
               if (gemm_float(part) != 0) return -1;
            }
            return 0;
         }
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
