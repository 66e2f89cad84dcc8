/* cfloat GEMM: as float, with real and imaginary planes (four real MFMAs per tile), K slab 8. */
#include "och_gemm.h"
namespace och {
int gemm_cfloat(const GemmArgs &g)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   switch (gemm_pick_tile(g, choice, 4))
   {  case 0:
         /* enough whole 128 x 128 tiles for every compute unit: these run on the pipelined kernel (och_gemm_c32p.hip), the
            strip of columns to their right and the strip of rows below them as products of their own */
         if (g.M >= 128 && g.N >= 128 && (uint64_t)(g.M / 128) * (g.N / 128) * g.nz >= (uint64_t)gemm_compute_units())
         {  const size_t Mi = g.M - g.M % 128, Ni = g.N - g.N % 128;
            GemmArgs part = g;
            part.M = Mi; part.N = Ni;
            const int taken = gemm_cfloat_pipe(part);
            if (taken < 0) return taken;
            if (taken == 0)
            {  if (g.N > Ni)
               {  part = g; part.N = g.N - Ni;
                  part.B = (const char *)g.B + (int64_t)Ni * (g.transB == 'N' ? (int64_t)g.ldB : 1) * 8;
                  part.C = (char *)g.C + (int64_t)Ni * g.ldC * 8;
                  if (gemm_cfloat(part) != 0) return -1;
               }
               if (g.M > Mi)
               {  part = g; part.M = g.M - Mi; part.N = Ni;
                  part.A = (const char *)g.A + (int64_t)Mi * (g.transA == 'N' ? 1 : (int64_t)g.ldA) * 8;
                  part.C = (char *)g.C + (int64_t)Mi * 8;
                  if (gemm_cfloat(part) != 0) return -1;
               }
               return 0;
            }
         }
         return launch_gemm_mfma<float, true, 64, 64, 8>(g);
      case 1:  return launch_gemm_mfma<float, true, 64, 32, 8>(g);
      case 2:  return launch_gemm_mfma<float, true, 32, 64, 8>(g);
      default: return launch_gemm_mfma<float, true, 32, 32, 8>(g);
   }
}
}
