/* float GEMM: block tiles of 128 x 128 (64 x 64 per wave, 2 x 2 tiles of 32x32x2), 128 x 64, 64 x 128 or 64 x 64, K slab 16;
   the tile is chosen by how well the tile count fills the rounds of the compute units (gemm_pick_tile). Efficiencies from
   4000^3: 106 / 100 / 97 / 91 TFLOP/s. */
#include "och_gemm.h"
namespace och {
/* Which kernel an aligned float product takes: 256, 128 or 64 (the pipelined kernel of och_gemm_f32p.hip on that tile) or
   0 (the tiled kernels below, tile number *pick). Host arithmetic only.
   Large and small tile against each other and against the tiled kernels by the model of gemm_pick_tile: rounds of the
   compute units x tile area / efficiency, with the tiled kernels at 0.8 of the pipelined kernel on 256 x 256 tiles and
   the 128 x 128 tiles at 0.95 (8192^3: 130 against 153 TFLOP/s; 2048^3: 84 against 135).
   Products of at most four rounds of 64 x 64 tiles (2048 x 2048 and below: what was measured) are priced in microseconds as well, from
   measurements of 512^3 ... 2048^3 and of 1024 x 1024 x 4096, 1024 x 2048 x 1024 and 2048 x 2048 x 512 (MI355X):
   a block of 64 x 64 takes 0.427 us per slab of 32 k at full rate and runs at 0.71 of that alone on its compute unit,
   0.88 with a second block beside it, 0.9 with more (the neighbours cover its waits); a block of 128 x 128 takes 1.8 us per
   slab, of 256 x 256 6.9 us; a launch costs 10 to 12 us before its first and after its last MFMA, and a tile cut along K
   13 us more (8 us on the smallest tile) for the shares' way through the workspace. The smallest tile is taken where it
   is the cheaper one by these figures, and wherever the model above would have sent the product to the tiled kernels
   (1024^3: 69 against 49 TFLOP/s; 1536^3: 107 against 75 on the 128 x 128 tile). */
static int gemm_float_plan(const GemmArgs &g, int *pick)
{  static const GemmTileChoice choice[4] = { { 128, 128, 1.0 }, { 128, 64, 0.94 }, { 64, 128, 0.94 }, { 64, 64, 0.86 } };
   *pick = gemm_pick_tile(g, choice, 4);
   if (!(g.M >= 128 && g.N >= 128 && g.M % 4 == 0 && g.N % 4 == 0 && g.K >= 32 && (g.K % 32 == 0 || (g.scalar_mode_host && g.K >= 256)))) return 0;
   const uint64_t units = (uint64_t)gemm_compute_units();
   auto cost = [&](uint64_t bm, uint64_t bn, double efficiency)
   {  const uint64_t tiles = ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * (uint64_t)g.nz;
      return (double)((tiles + units - 1) / units) * (double)(bm * bn) / efficiency;
   };
   /* the pipelined kernel cuts the tiles of a last round that is at most half full along K: that round then counts as
      1 / shares of a round */
   GemmArgs whole = g;
   whole.K = g.K - g.K % 32;
   double rounds_large = 0, rounds_small = 0;
   const int shares_large = gemm_float_pipe_split(whole, 256, &rounds_large), shares_small = gemm_float_pipe_split(whole, 128, &rounds_small);
   /* what a block spends outside its main loop, in slabs of 32 k: about three on the large tile and in the tiled
      kernels, two on the small tile (8192 x 8192 x 256: 109, 93 and 118 TFLOP/s) */
   const double slabs = (double)(whole.K / 32);
   const double large = rounds_large * 65536.0 * (slabs + 3) / slabs, small = rounds_small * 16384.0 / 0.95 * (slabs + 2) / slabs;
   const double others = cost(choice[*pick].bm, choice[*pick].bn, choice[*pick].efficiency * 0.8) * (slabs + 3) / slabs;
   const int forced = gemm_kernel_choice();
   if (forced == 1) return 256;
   if (forced == 2) return 128;
   if (forced == 3) return 0;
   if (forced == 4) return 64;
   int tile = large <= small ? 256 : 128;
   if (!((tile == 256 ? large : small) < others)) tile = 0;
   const uint64_t tiles64 = ((g.M + 63) / 64) * ((g.N + 63) / 64) * (uint64_t)g.nz;
   if (tiles64 <= 4 * units)
   {  if (tile == 0) return slabs <= 256 ? 64 : 0;      /* (measured up to K = 4096; a longer K stays where it was) */
      if (slabs <= 2) return tile;          /* the small tile has a kernel of its own for a K of one or two slabs */
      /* microseconds of a launch: `slab_us` per slab and block, the whole rounds, then the last round, cut or not */
      auto micros = [&](uint64_t edge, int shares, double fixed, double slab_us, double cut_us)
      {  const uint64_t tiles = ((g.M + edge - 1) / edge) * ((g.N + edge - 1) / edge) * (uint64_t)g.nz;
         const double last = tiles % units == 0 ? 0.0 : (shares > 1 ? (double)(((uint64_t)slabs + shares - 1) / shares) : slabs);
         return fixed + slab_us * ((double)(tiles / units) * slabs + last) + (shares > 1 ? cut_us : 0.0);
      };
      const int shares_smallest = gemm_float_pipe_split(whole, 64, nullptr);
      const double rate = tiles64 * (uint64_t)shares_smallest <= units ? 0.714 : (tiles64 <= 2 * units ? 0.88 : 0.9);
      const double smallest_us = micros(64, shares_smallest, 10.0, 0.427 / rate, 8.0);
      const double other_us = tile == 256 ? micros(256, shares_large, 12.0, 6.9, 13.0) : micros(128, shares_small, 12.0, 1.8, 13.0);
      if (smallest_us < other_us) return 64;
   }
   return tile;
}

int gemm_float(const GemmArgs &g)
{  int pick = 0;
   /* Aligned products with M and N multiples of 4 and K of 32 run on the pipelined kernel (och_gemm_f32p.hip) on tiles of
      256 x 256, 128 x 128 or 64 x 64 where gemm_float_plan finds that cheaper. A K that is not a multiple of 32 (scalars in
      host memory only): the whole slabs there, the rest of K as a product of its own that adds to C. */
   int tile = gemm_float_plan(g, &pick);
   if (!gemm_operands_aligned(g, 4)) tile = 0;
   if (tile != 0)
   {  static const float one = 1.0f;
      const int done = gemm_pipelined_head_and_rest(g, 32, 4, &one, [&](const GemmArgs &a) { return gemm_float_pipe(a, tile); }, gemm_float);
      if (done <= 0) return done;
   }
   switch (pick)
   {  case 0:  return launch_gemm_mfma<float, false, 64, 64, 16>(g);
      case 1:  return launch_gemm_mfma<float, false, 64, 32, 16>(g);
      case 2:  return launch_gemm_mfma<float, false, 32, 64, 16>(g);
      default: return launch_gemm_mfma<float, false, 32, 32, 16>(g);
   }
}

/* the plan of a single (batch = 1) or batched aligned product with scalars in host memory, for tests: no device is touched */
int gemm_float_plan_query(uint64_t M, uint64_t N, uint64_t K, unsigned batch)
{  GemmArgs g;
   memset(&g, 0, sizeof(g));
   g.M = M; g.N = N; g.K = K; g.ldA = (int64_t)M; g.ldB = (int64_t)K; g.ldC = (int64_t)M; g.transA = 'N'; g.transB = 'N';
   g.scalar_mode_host = 1; g.nz = batch == 0 ? 1 : batch;
   if (batch > 1) { g.batch.nb = 1; g.batch.size[0] = batch; }
   int pick = 0;
   return gemm_float_plan(g, &pick);
}
}
