/* float GEMM: block tiles of 128 x 128 (64 x 64 per wave, 2 x 2 tiles of 32x32x2), 128 x 64, 64 x 128 or 64 x 64, K slab 16;
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 106 / 100 / 97 / 91 TFLOP/s. Large aligned products with K a multiple of 32 run their whole 256 x 256 tiles on
   the pipelined kernel of och_gemm_f32p.hip (8192^3: 130 -> 153 TFLOP/s). */
#include "och_gemm.h"
namespace och {
int gemm_float(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   switch (gemm_pick_tile(g, choice, 4))
   {  case 0:
         /* enough whole 256 x 256 tiles for every compute unit: these run on the pipelined kernel (och_gemm_f32p.hip), the
            strip of columns to their right and the strip of rows below them as products of their own */
         if (g.M >= 256 && g.N >= 256 && (uint64_t)(g.M / 256) * (g.N / 256) * g.nz >= (uint64_t)gemm_compute_units())
         {  const size_t Mi = g.M - g.M % 256, Ni = g.N - g.N % 256;
            GemmArgs part = g;
            part.M = Mi; part.N = Ni;
            const int taken = gemm_float_pipe(part);
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
         return launch_gemm_mfma<float, false, 64, 64, 16>(g);
      case 1:  return launch_gemm_mfma<float, false, 64, 32, 16>(g);
      case 2:  return launch_gemm_mfma<float, false, 32, 64, 16>(g);
      default: return launch_gemm_mfma<float, false, 32, 32, 16>(g);
   }
}
}
