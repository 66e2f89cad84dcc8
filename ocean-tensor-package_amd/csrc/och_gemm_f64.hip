/* double GEMM: block tiles of 128 x 128 (64 x 64 per wave, 4 x 4 tiles of 16x16x4), 128 x 64, 64 x 128 or 64 x 64, K slab 16 (two barriers fewer per 16 k than with slabs of 8: 8192^3 TN 64.3 -> 66.1, NT 66.3 -> 68.4 TFLOP/s);
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 56 / 55 / 55 / 53 TFLOP/s. */
#include "och_gemm.h"
namespace och {
int gemm_double(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.96 }, { 64, 128, 0.96 }, { 64, 64, 0.92 } };
   const int pick = gemm_pick_tile(g, choice, 4);
   /* Large aligned products with K a multiple of 16: the whole 256 x 128 tiles run on the pipelined kernel, the strip of
      columns to their right and the strip of rows below them as products of their own -- when that is cheaper by the model
      of gemm_pick_tile (rounds of the compute units x tile area / efficiency, the kernels below at 0.87 of the pipelined one) */
   if (g.M >= 256 && g.N >= 128 && g.K >= 16 && g.K % 16 == 0 && gemm_operands_aligned(g, 8))
   {  const uint64_t units = (uint64_t)gemm_compute_units();
      auto cost = [&](uint64_t bm, uint64_t bn, double efficiency, bool whole)
      {  const uint64_t tiles = (whole ? (g.M / bm) * (g.N / bn) : ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn)) * (uint64_t)g.nz;
         return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
      };
      if (cost(256, 128, 1.0, true) < cost(choice[pick].bm, choice[pick].bn, choice[pick].efficiency * 0.87, false))
      {  const size_t Mi = g.M - g.M % 256, Ni = g.N - g.N % 128;
         GemmArgs part = g;
         part.M = Mi; part.N = Ni;
         const int taken = gemm_double_pipe(part);
         if (taken < 0) return taken;
         if (taken == 0)
         {  if (g.N > Ni)
            {  part = g; part.N = g.N - Ni;
               part.B = (const char *)g.B + (int64_t)Ni * (g.transB == 'N' ? (int64_t)g.ldB : 1) * 8;
               part.C = (char *)g.C + (int64_t)Ni * g.ldC * 8;
               if (gemm_double(part) != 0) return -1;
            }
            if (g.M > Mi)
            {  part = g; part.M = g.M - Mi; part.N = Ni;
               part.A = (const char *)g.A + (int64_t)Mi * (g.transA == 'N' ? 1 : (int64_t)g.ldA) * 8;
               part.C = (char *)g.C + (int64_t)Mi * 8;
               if (gemm_double(part) != 0) return -1;
            }
            return 0;
         }
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
