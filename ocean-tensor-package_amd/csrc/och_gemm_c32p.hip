/* complex float GEMM on tiles of 128 x 128 for aligned operands with M and N multiples of 2 and K of 32: C <- alpha * op(A) * op(B) + beta * C, column-major, op = none,
 * transposition or conjugate transposition.
 *
 * The counterpart of cublasCgemm in the reference (src/core/gpu/op/tensor_blas_gpu.c:183-197). The float kernel
 * (och_gemm_f32p.hip) with complex operands: four waves per block, one per SIMD, each owning 64 x 64 complex elements as
 * 2 x 2 tiles of 32 x 32, every tile with FOUR real accumulators -- Ar Br, Ai Bi, Ar Bi and Ai Br summed over k by
 * v_mfma_f32_32x32x2_f32 -- which are combined when C is written: the signs of the combination are all that conjugation
 * changes, and the matrix cores have no operand negation that the usual two accumulators would need. 16 accumulators of
 * 16 registers, 16 independent MFMAs per step, as in the float kernel; the main loop again holds MFMAs, LDS reads, scalar
 * instructions and loads that go from memory straight to LDS, and no vector arithmetic.
 *
 *   - a slab is 32 k of 128 rows, 32 KB per operand as in the float kernel. Elements stay interleaved (re, im). An operand
 *     that is contiguous along k in memory lies in LDS as 16-byte chunks of 2 k, chunk-major: [chunk][row][2 complex]; lane
 *     l of a load instruction fetches one chunk of row l of 64 rows. An operand that is contiguous along m / n lies in LDS
 *     as it lies in memory, [k][128 rows]; a load instruction fetches one k of all rows.
 *   - one 16-byte fragment read yields, for a k-contiguous operand, (re, im) of one tile for two steps; for the other
 *     kind, (re, im) of both tiles for one step, tile i then being the rows 2 r + i, which is undone when C is written.
 *     In step t of pair P (two steps) the lanes hold k = 4 P + 2 (l / 32) + t for both operands.
 *   - schedule, buffers, barrier and clamped loads are those of the float kernel: quads of four steps = 64 MFMAs = 32
 *     chunks of two; 8 fragment reads of the next quad and, in quads 3 and 0, 8 loads each, one to every fourth chunk.
 *   - C leaves through LDS in passes of 32 columns, so that memory sees 16-byte accesses along the columns of C.
 */
#include "och_gemm.h"
#include "och_gemm_c32p_slab.h"
#pragma clang diagnostic ignored "-Winline-asm"

namespace och {


#define OCH_CP_BM 128
#define OCH_CP_KT 32
#define OCH_CP_THREADS 256
#define OCH_CP_BUFFER (2 * OCH_CP_OPERAND)

struct CFloatPipeParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   float    alpha[2], beta[2];          /* (re, im) */
   const float *alpha_dev, *beta_dev;
   int      conjA, conjB;
   uint32_t tiles_m, tiles_n;
   /* the tiles of the last, partly filled round of the compute units are cut along K: tiles from split_first on are
      computed by `split` blocks each, block q of them (counted from the first such block) leaving the raw complex sums of
      its share of the slabs in partial[q] (a dense tile, column-major); the finish kernel adds the shares in order and
      applies alpha / beta. split <= 1: no tile is cut. Only without a batch. */
   uint32_t split_first, split;
   float *partial;
   GemmBatch batch;
};

template <bool AKC, bool BKC>
__global__ __launch_bounds__(OCH_CP_THREADS) void gemm_cfloat_pipe_kernel(const CFloatPipeParams p)
{
   constexpr int T = 32, BM = OCH_CP_BM, BN = OCH_CP_BM, KT = OCH_CP_KT, TMS = 2, TNS = 2, WM = 64, WN = 64, THREADS = OCH_CP_THREADS;
   constexpr uint32_t OP = OCH_CP_OPERAND, BUF = OCH_CP_BUFFER;
   typedef CFloatSlab<AKC> LA;
   typedef CFloatSlab<BKC> LB;
   extern __shared__ __align__(16) char lds[];

   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const char *pA = p.A + oA, *pB = p.B + oB; char *pC = p.C + oC;
   uint32_t tile = blockIdx.x, share = 0, shares = 1, cut = 0;           /* cut: index of this block among those of cut tiles */
   if (p.split > 1 && blockIdx.x >= p.split_first)
   {  cut = blockIdx.x - p.split_first; tile = p.split_first + cut / p.split; share = cut % p.split; shares = p.split; }
   const uint32_t tile_m = tile % p.tiles_m, tile_n = tile / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
   const uint32_t wm = (wave % 2) * WM, wn = (wave / 2) * WN;

   och_f32x16 acc[TMS][TNS][4];            /* per tile: sums of Ar Br, Ai Bi, Ar Bi, Ai Br */
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
#pragma unroll
         for (int a = 0; a < 4; a++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][a][r] = 0;

   /* this block's slabs: slab0 .. last of the product's K / KT (all of them unless the tile is cut) */
   const uint32_t per_share = (p.K / KT + shares - 1) / shares, slab0 = share * per_share;
   const uint32_t nslabs = slab0 + per_share <= p.K / KT ? per_share : p.K / KT - slab0, last = slab0 + nslabs - 1;
   const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)lds;      /* where the array starts in LDS */
   const uint32_t rowsA = p.M - m0 < (uint32_t)BM ? p.M - m0 : (uint32_t)BM, rowsB = p.N - n0 < (uint32_t)BN ? p.N - n0 : (uint32_t)BN;    /* of this tile */
   uint32_t offA[8], offB[8], tgtA[8], tgtB[8];
#pragma unroll
   for (int j = 0; j < 8; j++)
   {  offA[j] = LA::load_offset(j, wave, lane, p.ldA, rowsA); offB[j] = LB::load_offset(j, wave, lane, p.ldB, rowsB);
      tgtA[j] = lds0 + LA::load_target(j, wave); tgtB[j] = lds0 + OP + LB::load_target(j, wave);
   }
   /* the lane's read addresses in buffer 0 and buffer 1, in registers of their own (the empty asm keeps the compiler
      from deriving the second from the first with an addition at every read: the distance is beyond a read's immediate) */
   const char *readA[2], *readB[2];
   {  uint32_t a1 = LA::read_lane(wm, lane) + BUF, b1 = OP + LB::read_lane(wn, lane) + BUF;
      asm volatile("" : "+v"(a1), "+v"(b1));
      readA[0] = lds + LA::read_lane(wm, lane); readA[1] = lds + a1;
      readB[0] = lds + OP + LB::read_lane(wn, lane); readB[1] = lds + b1;
   }
   och_f32x4 fa[2][4], fb[2][4];

   /* load number e (0 .. 15; A first) of slab `slab` into buffer `buf` */
#define OCH_LOAD(e, baseA, baseB, buf)                                                                                 \
   do { if ((e) < 8) load_to_lds(baseA, offA[(e) % 8], tgtA[(e) % 8] + (buf) * BUF);                                   \
        else         load_to_lds(baseB, offB[(e) % 8], tgtB[(e) % 8] + (buf) * BUF); } while (0)
   /* one quad: chunk c reads fragment c / 4 of quad QN from buffer RB into set NXT when c is a multiple of four, issues
      load LOAD0 + c / 4 into buffer LBUF when c % 4 == 2 and LOADS is set, then runs its two MFMAs */
#define OCH_QUAD(CUR, NXT, RB, QN, LOADS, LOAD0, LBUF)                                                                 \
   do { _Pragma("unroll") for (int c = 0; c < 32; c++)                                                                \
        {  if (c % 4 == 0)                                                                                             \
           {  if (c / 4 < 4) fa[NXT][c / 4 % 4] = *reinterpret_cast<const och_f32x4 *>(readA[RB] + LA::read_offset(c / 4 % 4, QN)); \
              else           fb[NXT][c / 4 % 4] = *reinterpret_cast<const och_f32x4 *>(readB[RB] + LB::read_offset(c / 4 % 4, QN)); \
           }                                                                                                           \
           if (LOADS && c % 4 == 2) OCH_LOAD(LOAD0 + c / 4, nextA, nextB, LBUF);                                       \
           {  const int st = c / 8, i = (c % 8) / 4, j = (c % 8) / 2 % 2, ci = c % 2;     /* A's real part, then its imaginary part */ \
              acc[i][j][ci] = __builtin_amdgcn_mfma_f32_32x32x2f32(LA::value(fa[CUR], i, st, ci), LB::value(fb[CUR], j, st, ci), acc[i][j][ci], 0, 0, 0); \
              acc[i][j][2 + ci] = __builtin_amdgcn_mfma_f32_32x32x2f32(LA::value(fa[CUR], i, st, ci), LB::value(fb[CUR], j, st, 1 - ci), acc[i][j][2 + ci], 0, 0, 0); \
           }                                                                                                           \
           __builtin_amdgcn_sched_barrier(0);                                                                          \
        } } while (0)
   /* slab s in buffer CB: quad 0 carries the second half of the loads of slab s + 1 (into the other buffer), quad 3 the
      first half of the loads of slab s + 2 (into this one) */
#define OCH_SLAB(s, CB)                                                                                                \
   do { {  const uint32_t s1 = (slab0 + (s) + 1 < last) ? slab0 + (s) + 1 : last;                                                      \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);  \
           OCH_QUAD(0, 1, CB, 1, true, 8, 1 - CB);                                                                     \
        }                                                                                                              \
        {  const char *nextA = nullptr, *nextB = nullptr;                                                              \
           OCH_QUAD(1, 0, CB, 2, false, 0, 0);                                                                         \
           OCH_QUAD(0, 1, CB, 3, false, 0, 0);                                                                         \
        }                                                                                                              \
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                               \
        __syncthreads();                                                                                               \
        {  const uint32_t s2 = (slab0 + (s) + 2 < last) ? slab0 + (s) + 2 : last;                                                      \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);  \
           OCH_QUAD(1, 0, 1 - CB, 0, true, 0, CB);                                                                     \
        } } while (0)

   {  /* slab 0 and the first half of slab 1 */
      const uint32_t s1 = (slab0 + 1 < last) ? slab0 + 1 : last;
      const char *nextA = LA::slab_base(pA, p.ldA, m0, slab0 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, slab0 * KT);
#pragma unroll
      for (int e = 0; e < 16; e++) OCH_LOAD(e, nextA, nextB, 0);
      nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT); nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);
#pragma unroll
      for (int e = 0; e < 8; e++) OCH_LOAD(e, nextA, nextB, 1);
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      __syncthreads();
#pragma unroll
      for (int x = 0; x < 4; x++)
      {  fa[0][x] = *reinterpret_cast<const och_f32x4 *>(readA[0] + LA::read_offset(x, 0));
         fb[0][x] = *reinterpret_cast<const och_f32x4 *>(readB[0] + LB::read_offset(x, 0));
      }
   }
   uint32_t s = 0;
   for (; s + 1 < nslabs; s += 2)
   {  OCH_SLAB(s, 0);
      OCH_SLAB(s + 1, 1);
   }
   if (s < nslabs) OCH_SLAB(s, 0);
   asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
   __syncthreads();
#undef OCH_SLAB
#undef OCH_QUAD
#undef OCH_LOAD

   /* epilogue: accumulator register r of lane l is row-in-tile 8 * (r / 4) + 4 * (l / 32) + r % 4 of A's tile and
      row-in-tile l % 32 of B's. Real part Ar Br -+ Ai Bi, imaginary part +- Ar Bi +- Ai Br, the signs by the conjugations.
      The scaled tile goes through LDS, 32 columns at a time with a pitch of BM + 2 elements, and leaves (after beta * C has
      been added) in 16-byte pieces that follow the columns of C. */
   float ar = p.alpha[0], ai = p.alpha[1], br = p.beta[0], bi = p.beta[1];
   if (p.alpha_dev) { const float *q = reinterpret_cast<const float *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha); ar = q[0]; ai = q[1]; }
   if (p.beta_dev)  { const float *q = reinterpret_cast<const float *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta); br = q[0]; bi = q[1]; }
   const float sq = (p.conjA != p.conjB) ? 1.0f : -1.0f, s1 = p.conjB ? -1.0f : 1.0f, s2 = p.conjA ? -1.0f : 1.0f;
   /* a share of a cut tile leaves its raw sums, the whole tile, in the workspace */
   char *out = pC + ((int64_t)m0 + (int64_t)n0 * p.ldC) * 8;
   int64_t ldOut = p.ldC;
   uint32_t rowsOut = rowsA, colsOut = rowsB;
   if (shares > 1)
   {  ar = 1; ai = 0; br = 0; bi = 0;
      out = reinterpret_cast<char *>(p.partial + (size_t)cut * BM * BN * 2); ldOut = BM; rowsOut = BM; colsOut = BN;
   }
   constexpr int CP = BM + 2, CPASS = 32, PASSES = BN / CPASS;
   static_assert(CPASS * CP * 8 <= 2 * BUF, "a pass of the staged tile does not fit into the slab buffers");
   float2 *stage = reinterpret_cast<float2 *>(lds);
   for (int h = 0; h < PASSES; h++)
   {
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {  const uint32_t col = wn + LB::row(j, lane % T);
         if (col / CPASS != (uint32_t)h) continue;
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {  const float cr = acc[i][j][0][r] + sq * acc[i][j][1][r], ci = s1 * acc[i][j][2][r] + s2 * acc[i][j][3][r];
               stage[(col - h * CPASS) * CP + wm + LA::row(i, 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3))] = make_float2(ar * cr - ai * ci, ar * ci + ai * cr);
            }
      }
      __syncthreads();
      for (uint32_t q = threadIdx.x; q < CPASS * (BM / 2); q += THREADS)
      {  const uint32_t c = q / (BM / 2), r2 = (q % (BM / 2)) * 2;
         if (r2 >= rowsOut || h * CPASS + c >= colsOut) continue;      /* outside C */
         och_f32x4 v = *reinterpret_cast<const och_f32x4 *>(stage + c * CP + r2);
         och_f32x4 *dst = reinterpret_cast<och_f32x4 *>(out + ((int64_t)r2 + (int64_t)(h * CPASS + c) * ldOut) * 8);
         if (br != 0 || bi != 0)
         {  const och_f32x4 old = *dst;
            v.x += br * old.x - bi * old.y; v.y += br * old.y + bi * old.x;
            v.z += br * old.z - bi * old.w; v.w += br * old.w + bi * old.z;
         }
         *dst = v;
      }
      __syncthreads();
   }
}

/* The shares of the cut tiles, added in the order of their slabs, times alpha, plus beta * C: a block per 16 columns of a
   cut tile (grid y), one element of C per thread and trip. */
__global__ __launch_bounds__(256) void gemm_cfloat_pipe_finish_kernel(const CFloatPipeParams p)
{
   constexpr uint32_t BM = 128, BN = 128;
   const uint32_t tile = p.split_first + blockIdx.x, tile_m = tile % p.tiles_m, tile_n = tile / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const uint32_t rows = p.M - m0 < BM ? p.M - m0 : BM, cols = p.N - n0 < BN ? p.N - n0 : BN;
   const float ar = p.alpha_dev ? p.alpha_dev[0] : p.alpha[0], ai = p.alpha_dev ? p.alpha_dev[1] : p.alpha[1];
   const float br = p.beta_dev ? p.beta_dev[0] : p.beta[0], bi = p.beta_dev ? p.beta_dev[1] : p.beta[1];
   const float *shares = p.partial + (size_t)blockIdx.x * p.split * BM * BN * 2;
   for (uint32_t q = threadIdx.x; q < 16 * BM; q += 256)
   {  const uint32_t c = blockIdx.y * 16 + q / BM, r = q % BM;
      if (r >= rows || c >= cols) continue;
      float sr = 0, si = 0;
      for (uint32_t t = 0; t < p.split; t++)
      {  const float *w = shares + ((size_t)t * BM * BN + (size_t)c * BM + r) * 2;
         sr += w[0]; si += w[1];
      }
      float vr = ar * sr - ai * si, vi = ar * si + ai * sr;
      float *dst = reinterpret_cast<float *>(p.C + ((int64_t)(m0 + r) + (int64_t)(n0 + c) * p.ldC) * 8);
      if (br != 0 || bi != 0) { const float cr = dst[0], ci = dst[1]; vr += br * cr - bi * ci; vi += br * ci + bi * cr; }
      dst[0] = vr; dst[1] = vi;
   }
}

/* Into how many shares the tiles of the last round are cut (1: not at all): the round must be at most half full, every
   share at least 8 slabs long, at most 8 shares per tile (64 when the whole product is less than one round), and all shares must fit into the stream's workspace. *rounds: the rounds of the compute
   units the product then takes (for the cost model of the caller); the cut round counts as the length of a share plus
   what every block spends outside its main loop (about 6 slabs' worth) over the length of a whole tile. */
int gemm_cfloat_pipe_split(const GemmArgs &g, double *rounds)
{
   return gemm_pipe_split_plan(g.M, g.N, g.K, (uint64_t)g.nz, g.batch.nb == 0, 128, 128, 32, 8, (uint64_t)gemm_compute_units(), rounds);
}

/* 0: launched; 1: not a case for this kernel (the caller's other kernels take it) */
int gemm_cfloat_pipe(const GemmArgs &g)
{
   if (g.M % 2 != 0 || g.N % 2 != 0 || g.M == 0 || g.N == 0 || g.K % OCH_CP_KT != 0 || g.K == 0 || !gemm_operands_aligned(g, 8)) return 1;
   /* a lane's offset within a slab (up to 127 columns further on) is kept in 32 bits */
   if ((int64_t)g.ldA * 8 >= (1 << 24) || (int64_t)g.ldB * 8 >= (1 << 24)) return 1;
   CFloatPipeParams p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host) { memcpy(p.alpha, g.alpha, 8); memcpy(p.beta, g.beta, 8); }
   else { p.alpha_dev = (const float *)g.alpha; p.beta_dev = (const float *)g.beta; }
   p.batch = g.batch;
   p.conjA = (g.transA == 'C'); p.conjB = (g.transB == 'C');
   p.tiles_m = (uint32_t)((g.M + OCH_CP_BM - 1) / OCH_CP_BM); p.tiles_n = (uint32_t)((g.N + OCH_CP_BM - 1) / OCH_CP_BM);
   uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   const int shares = gemm_cfloat_pipe_split(g, nullptr);
   uint32_t cut_tiles = 0;
   if (shares > 1)
   {  char *ws;
      if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
      cut_tiles = (uint32_t)(blocks % (uint64_t)gemm_compute_units());
      p.split = (uint32_t)shares; p.split_first = (uint32_t)blocks - cut_tiles; p.partial = reinterpret_cast<float *>(ws);
      blocks += (uint64_t)cut_tiles * (shares - 1);
   }
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   const dim3 grid((unsigned)blocks, 1, g.nz), block(OCH_CP_THREADS);
   const size_t lds = 2 * (size_t)OCH_CP_BUFFER;
#define OCH_CP_LAUNCH(AK, BK)                                                                                         \
   do { auto kernel = gemm_cfloat_pipe_kernel<AK, BK>;                                                                 \
        OCH_CHECK_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kernel, grid, block, lds, g.stream, p); } while (0)
   if (!akc && !bkc) OCH_CP_LAUNCH(false, false);
   else if (!akc)    OCH_CP_LAUNCH(false, true);
   else if (!bkc)    OCH_CP_LAUNCH(true, false);
   else              OCH_CP_LAUNCH(true, true);
#undef OCH_CP_LAUNCH
   if (shares > 1) hipLaunchKernelGGL(gemm_cfloat_pipe_finish_kernel, dim3(cut_tiles, 8), dim3(256), 0, g.stream, p);
   OCH_CHECK_LAUNCH();
   return 0;
}

} /* namespace och */
