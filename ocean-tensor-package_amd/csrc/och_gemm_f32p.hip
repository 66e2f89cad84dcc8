/* float GEMM on tiles of 256 x 256, 128 x 128 or 64 x 64 for aligned operands with M and N multiples of 4 and K of 32: C <- alpha * op(A) * op(B) + beta * C, column-major.
 *
 * The counterpart of cublasSgemm in the reference (src/core/gpu/op/tensor_blas_gpu.c:183-197). Four waves per block,
 * one per SIMD, each owning 128 x 128 of the tile as 4 x 4 tiles of v_mfma_f32_32x32x2_f32 (256 accumulator registers);
 * for products with fewer than one such tile per compute unit the same kernel with TS = 2: waves of 64 x 64 (2 x 2
 * tiles), two blocks per compute unit (SINGLE: one slab buffer of 34 KB and about a hundred registers, four blocks, for a K of one or two slabs);
 * for products of a few hundred tiles at most, TS = 1: waves of 32 x 32 (one tile, a chunk being two steps of it), 36 KB
 * of LDS and under 48 registers, up to four blocks per compute unit (1024^3: 69 TFLOP/s against 53 on the 128 x 128 tile,
 * whose 64 tiles have to be cut along K; 1536^3: 107 against 75). With one block on a compute unit its loads have only
 * three quads of four MFMAs (770 cycles) to arrive and the block waits for them: it runs at 0.7 of the matrix rate, at 0.9
 * with a second block beside it. NB = 4 would keep four slab buffers in a ring instead of two, so that a load has three
 * slabs to arrive; the kernel is written for it, but that form has not run on a device and is not instantiated.
 * The description is for TS = 4.
 * On this device a vector-ALU instruction of a wave takes about eight cycles away from the matrix cores of its SIMD, and
 * a 64-cycle MFMA hides none of that; LDS reads and scalar instructions are nearly free. So the main loop holds MFMAs,
 * LDS reads, scalar instructions and loads that go from memory straight to LDS -- no vector arithmetic, no staging
 * registers, no LDS stores:
 *
 *   - a slab is 32 k. An operand that is contiguous along k in memory ("k-contiguous": A of a T product, B of an N
 *     product) lies in LDS as 16-byte chunks of 4 k, chunk-major: [chunk][row][4 floats]; lane l of a load instruction
 *     fetches one chunk of row l of the wave's 64 rows. An operand that is contiguous along m / n lies in LDS as it
 *     lies in memory, [k][256 rows]; a load instruction fetches one k of all 256 rows. Either way the 64 lanes of a load
 *     write 1 KB of consecutive LDS, which is what loads to LDS do (M0 holds the address, the lanes follow each other).
 *   - an MFMA step consumes one float per lane and operand (lanes 0-31: one k, lanes 32-63: another). One 16-byte
 *     fragment read yields, for a k-contiguous operand, the values of one 32-row tile for four steps; for the other
 *     kind, the values of four tiles for one step, the tiles then being made of every fourth row (tile i = rows 4 r + i),
 *     which is undone when C is written. Four steps are a "quad"; in step t of quad q the lanes hold k = 8 q + 4 (l / 32) + t
 *     for both operands.
 *   - a quad is 64 MFMAs = 32 chunks of two, each closed by a scheduling fence; the 8 fragment reads of the NEXT quad go
 *     one to every fourth chunk (two sets of fragment registers). The one barrier of a slab stands in front of quad 3,
 *     behind a wait for the wave's own loads: after it slab s + 1 is complete in the other buffer (quad 3 reads its
 *     first fragments) and nobody reads the rest of this buffer again, so quad 3 and quad 0 of the next slab issue the
 *     16 loads of slab s + 2 into it, one to every fourth chunk. A load has three quads (12000 cycles) to arrive.
 *   - the loop body has no branches: slab numbers past the end are clamped (the last slab is loaded again into a buffer
 *     nobody reads); it is written out twice so that all LDS offsets are immediates.
 *   - C leaves through LDS in passes of 64 columns, so that memory sees 16-byte accesses along the columns of C.
 *   - the last tiles of a matrix whose size is not a multiple of the tile: lanes whose rows do not exist load the last
 *     rows that do (every load stays inside the matrix, the loop is unchanged), and what lies outside C is not written.
 *   - the compute units work through the tiles in rounds, and a last round of a few tiles would take as long as a full
 *     one: when it is at most half full its tiles are cut along K into shares that fill it, each share leaves its raw sums
 *     in the stream's workspace, and gemm_float_pipe_finish_kernel adds them in slab order and applies alpha and beta.
 */
#include "och_gemm.h"
#include "och_gemm_f32p_slab.h"
#pragma clang diagnostic ignored "-Winline-asm"

namespace och {


#define OCH_FP_KT 32
#define OCH_FP_THREADS 256

struct FloatPipeParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   float    alpha, beta;
   const float *alpha_dev, *beta_dev;
   uint32_t tiles_m, tiles_n;
   /* the tiles of the last, partly filled round of the compute units are cut along K: tiles from split_first on are
      computed by `split` blocks each, block q of them (counted from the first such block) leaving the raw sums of its
      share of the slabs in partial[q] (a dense tile, column-major); gemm_float_pipe_finish_kernel adds the shares in
      order and applies alpha / beta. split <= 1: no tile is cut. Only without a batch. */
   uint32_t split_first, split;
   float   *partial;
   GemmBatch batch;
};

template <bool AKC, bool BKC, int TS, bool SINGLE = false, int NB = 2>
__global__ __launch_bounds__(OCH_FP_THREADS, TS == 4 ? 1 : (SINGLE || TS == 1 ? 4 : 2)) void gemm_float_pipe_kernel(const FloatPipeParams p)
{
   constexpr int T = 32, BM = 64 * TS, BN = 64 * TS, KT = OCH_FP_KT, TMS = TS, TNS = TS, WM = 32 * TS, WN = 32 * TS, THREADS = OCH_FP_THREADS;
   typedef FloatSlab<AKC, BM> LA;
   typedef FloatSlab<BKC, BN> LB;
   constexpr uint32_t OP = LA::OPERAND, BUF = 2 * OP;
   constexpr int NLA = LA::LOADS, NL = 2 * NLA;            /* loads per wave and slab: of A, of both */
   constexpr int CH = 2 * TS * TS;                         /* chunks of two MFMAs per quad */
   constexpr int RA = LA::READS, NR = LA::READS + LB::READS; /* fragment reads per quad: of A, of both */
   static_assert(TS == 4 || TS == 2 || TS == 1, "wave tiles of 128 x 128, 64 x 64 or 32 x 32");
   static_assert(NB == 2 || (NB == 4 && !SINGLE && BUF + 2 * OP < 65536), "two slab buffers, or a ring of four within reach of the immediates of two read addresses");
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

   och_f32x16 acc[TMS][TNS];
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
#pragma unroll
         for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

   /* this block's slabs: slab0 .. last of the product's K / KT (all of them unless the tile is cut) */
   const uint32_t per_share = (p.K / KT + shares - 1) / shares, slab0 = share * per_share;
   const uint32_t nslabs = slab0 + per_share <= p.K / KT ? per_share : p.K / KT - slab0, last = slab0 + nslabs - 1;
   const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)lds;      /* where the array starts in LDS */
   const uint32_t rowsA = p.M - m0 < (uint32_t)BM ? p.M - m0 : (uint32_t)BM, rowsB = p.N - n0 < (uint32_t)BN ? p.N - n0 : (uint32_t)BN;    /* of this tile */
   uint32_t offA[NLA], offB[NLA], tgtA[NLA], tgtB[NLA];
#pragma unroll
   for (int j = 0; j < NLA; j++)
   {  offA[j] = LA::load_offset(j, wave, lane, p.ldA, rowsA); offB[j] = LB::load_offset(j, wave, lane, p.ldB, rowsB);
      tgtA[j] = lds0 + LA::load_target(j, wave); tgtB[j] = lds0 + OP + LB::load_target(j, wave);
   }
   /* the lane's read addresses in buffer 0 and buffer 1, in registers of their own (the empty asm keeps the compiler
      from deriving the second from the first with an addition at every read: the distance is beyond a read's immediate) */
   const char *readA[2], *readB[2];
   {  uint32_t a1 = LA::read_lane(wm, lane) + (NB / 2) * BUF, b1 = OP + LB::read_lane(wn, lane) + (NB / 2) * BUF;
      asm volatile("" : "+v"(a1), "+v"(b1));
      readA[0] = lds + LA::read_lane(wm, lane); readA[1] = lds + a1;
      readB[0] = lds + OP + LB::read_lane(wn, lane); readB[1] = lds + b1;
   }
   och_f32x4 fa[2][4], fb[2][4];

   /* load number e (0 .. NL - 1; A's first) of a slab into buffer `buf` */
#define OCH_LOAD(e, baseA, baseB, buf)                                                                                 \
   do { if ((e) < NLA) load_to_lds(baseA, offA[(e) % NLA], tgtA[(e) % NLA] + (buf) * BUF);                             \
        else           load_to_lds(baseB, offB[(e) % NLA], tgtB[(e) % NLA] + (buf) * BUF); } while (0)
   /* one quad of CH chunks: chunk c issues its share of the NR fragment reads of quad QN from buffer RB into set NXT, and,
      when LOADS is set and c % TS == TS / 2, load LOAD0 + c / TS into buffer LBUF; then it runs its two MFMAs */
#define OCH_QUAD(CUR, NXT, RB, QN, LOADS, LOAD0, LBUF)                                                                 \
   do { _Pragma("unroll") for (int c = 0; c < CH; c++)                                                                \
        {  _Pragma("unroll") for (int f = c * NR / CH; f < (c + 1) * NR / CH; f++)                                     \
           {  if (f < RA) fa[NXT][f < RA ? f : 0] = LA::read(readA[(RB) / (NB / 2)] + ((RB) % (NB / 2)) * BUF + LA::read_offset(f < RA ? f : 0, QN)); \
              else        fb[NXT][f >= RA ? f - RA : 0] = LB::read(readB[(RB) / (NB / 2)] + ((RB) % (NB / 2)) * BUF + LB::read_offset(f >= RA ? f - RA : 0, QN)); \
           }                                                                                                           \
           if (LOADS && c % TS == TS / 2) OCH_LOAD(LOAD0 + c / TS, nextA, nextB, LBUF);                                \
           _Pragma("unroll") for (int x = 2 * c; x < 2 * c + 2; x++)                                                   \
           {  const int st = x / (TMS * TNS), i = x % (TMS * TNS) / TNS, j = x % TNS;                                  \
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(LA::value(fa[CUR], i, st), LB::value(fb[CUR], j, st), acc[i][j], 0, 0, 0); \
           }                                                                                                           \
           __builtin_amdgcn_sched_barrier(0);                                                                          \
        } } while (0)
   /* slab s in buffer CB: quad 0 carries the second half of the loads of slab s + 1 (into the other buffer), quad 3 the
      first half of the loads of slab s + 2 (into this one) */
#define OCH_SLAB(s, CB)                                                                                                \
   do { {  const uint32_t s1 = (slab0 + (s) + (NB - 1) < last) ? slab0 + (s) + (NB - 1) : last;                        \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);  \
           OCH_QUAD(0, 1, CB, 1, true, NL / 2, ((CB) + NB - 1) % NB);                                                  \
        }                                                                                                              \
        {  const char *nextA = nullptr, *nextB = nullptr;                                                              \
           OCH_QUAD(1, 0, CB, 2, false, 0, 0);                                                                         \
           OCH_QUAD(0, 1, CB, 3, false, 0, 0);                                                                         \
        }                                                                                                              \
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NB - 2) * NL) : "memory");                                         \
        __syncthreads();                                                                                               \
        {  const uint32_t s2 = (slab0 + (s) + NB < last) ? slab0 + (s) + NB : last;                                    \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);  \
           OCH_QUAD(1, 0, ((CB) + 1) % NB, 0, true, 0, CB);                                                            \
        } } while (0)

   if constexpr (SINGLE)
   {  /* one slab buffer, four blocks per compute unit: a block's loads are not covered by its own MFMAs but by those of
         its neighbours. For a K of a few slabs, where a block spends as long on its first loads and on writing C as in
         its loop. */
      for (uint32_t s = 0; s < nslabs; s++)
      {  const char *nextA = LA::slab_base(pA, p.ldA, m0, (slab0 + s) * KT), *nextB = LB::slab_base(pB, p.ldB, n0, (slab0 + s) * KT);
         if (s > 0) __syncthreads();
#pragma unroll
         for (int e = 0; e < NL; e++) OCH_LOAD(e, nextA, nextB, 0);
         asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
         __syncthreads();
#pragma unroll
         for (int x = 0; x < LA::READS; x++) fa[0][x] = LA::read(readA[0] + LA::read_offset(x, 0));
#pragma unroll
         for (int x = 0; x < LB::READS; x++) fb[0][x] = LB::read(readB[0] + LB::read_offset(x, 0));
         OCH_QUAD(0, 1, 0, 1, false, 0, 0);
         OCH_QUAD(1, 0, 0, 2, false, 0, 0);
         OCH_QUAD(0, 1, 0, 3, false, 0, 0);
         OCH_QUAD(1, 0, 0, 0, false, 0, 0);            /* (its reads are not used) */
      }
      __syncthreads();
   }
   else
   {
   {  /* slabs 0 .. NB - 2 and the first half of slab NB - 1 */
      const uint32_t s1 = (slab0 + (NB - 1) < last) ? slab0 + (NB - 1) : last;
      const char *nextA, *nextB;
#pragma unroll
      for (int b = 0; b < NB - 1; b++)
      {  const uint32_t sb = (b == 0 || slab0 + b < last) ? slab0 + b : last;
         nextA = LA::slab_base(pA, p.ldA, m0, sb * KT); nextB = LB::slab_base(pB, p.ldB, n0, sb * KT);
#pragma unroll
         for (int e = 0; e < NL; e++) OCH_LOAD(e, nextA, nextB, b);
      }
      nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT); nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);
#pragma unroll
      for (int e = 0; e < NL / 2; e++) OCH_LOAD(e, nextA, nextB, NB - 1);
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"((NB - 2) * NL + NL / 2) : "memory");
      __syncthreads();
#pragma unroll
      for (int x = 0; x < LA::READS; x++) fa[0][x] = LA::read(readA[0] + LA::read_offset(x, 0));
#pragma unroll
      for (int x = 0; x < LB::READS; x++) fb[0][x] = LB::read(readB[0] + LB::read_offset(x, 0));
   }
   uint32_t s = 0;
   if constexpr (NB == 2)
   {  for (; s + 1 < nslabs; s += 2)
      {  OCH_SLAB(s, 0);
         OCH_SLAB(s + 1, 1);
      }
      if (s < nslabs) OCH_SLAB(s, 0);
   }
   else
   {  for (; s + 3 < nslabs; s += 4)
      {  OCH_SLAB(s, 0);
         OCH_SLAB(s + 1, 1);
         OCH_SLAB(s + 2, 2 % NB);
         OCH_SLAB(s + 3, 3 % NB);
      }
      if (s < nslabs) OCH_SLAB(s, 0);
      if (s + 1 < nslabs) OCH_SLAB(s + 1, 1);
      if (s + 2 < nslabs) OCH_SLAB(s + 2, 2 % NB);
   }
   asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
   __syncthreads();
   }
#undef OCH_SLAB
#undef OCH_QUAD
#undef OCH_LOAD

   /* epilogue: accumulator register r of lane l is row-in-tile 8 * (r / 4) + 4 * (l / 32) + r % 4 of A's tile and
      row-in-tile l % 32 of B's. The scaled tile goes through LDS, 64 columns at a time with a pitch of BM + 4 floats, and
      leaves (after beta * C has been added) in 16-byte pieces that follow the columns of C. */
   float alpha = p.alpha, beta = p.beta;
   if (p.alpha_dev) alpha = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha);
   if (p.beta_dev)  beta = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);
   /* a share of a cut tile leaves its raw sums, the whole tile, in the workspace */
   char *out = pC + ((int64_t)m0 + (int64_t)n0 * p.ldC) * 4;
   int64_t ldOut = p.ldC;
   uint32_t rowsOut = rowsA, colsOut = rowsB;
   if (shares > 1)
   {  alpha = 1.0f; beta = 0.0f;
      out = reinterpret_cast<char *>(p.partial + (size_t)cut * BM * BN); ldOut = BM; rowsOut = BM; colsOut = BN;
   }
   constexpr int CP = BM + 4, CPASS = 64, PASSES = BN / CPASS;
   static_assert(CPASS * CP * 4 <= (SINGLE ? 1 : NB) * BUF, "a pass of the staged tile does not fit into the slab buffers");
   float *stage = reinterpret_cast<float *>(lds);
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
               stage[(col - h * CPASS) * CP + wm + LA::row(i, 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3))] = alpha * acc[i][j][r];
      }
      __syncthreads();
      for (uint32_t q = threadIdx.x; q < CPASS * (BM / 4); q += THREADS)
      {  const uint32_t c = q / (BM / 4), r4 = (q % (BM / 4)) * 4;
         if (r4 >= rowsOut || h * CPASS + c >= colsOut) continue;      /* outside C */
         och_f32x4 v = *reinterpret_cast<const och_f32x4 *>(stage + c * CP + r4);
         och_f32x4 *dst = reinterpret_cast<och_f32x4 *>(out + ((int64_t)r4 + (int64_t)(h * CPASS + c) * ldOut) * 4);
         if (beta != 0) { const och_f32x4 old = *dst; v.x += beta * old.x; v.y += beta * old.y; v.z += beta * old.z; v.w += beta * old.w; }
         *dst = v;
      }
      __syncthreads();
   }
}

/* The shares of the cut tiles, added in the order of their slabs, times alpha, plus beta * C: a block per 32 columns of a
   cut tile (grid y), 16 bytes of a column of C per thread and trip. */
template <int TS>
__global__ __launch_bounds__(256) void gemm_float_pipe_finish_kernel(const FloatPipeParams p)
{
   constexpr uint32_t BM = 64 * TS, BN = 64 * TS;
   const uint32_t tile = p.split_first + blockIdx.x, tile_m = tile % p.tiles_m, tile_n = tile / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const uint32_t rows = p.M - m0 < BM ? p.M - m0 : BM, cols = p.N - n0 < BN ? p.N - n0 : BN;
   const float alpha = p.alpha_dev ? *p.alpha_dev : p.alpha, beta = p.beta_dev ? *p.beta_dev : p.beta;
   const float *shares = p.partial + (size_t)blockIdx.x * p.split * BM * BN;
   for (uint32_t q = threadIdx.x; q < 32 * (BM / 4); q += 256)
   {  const uint32_t c = blockIdx.y * 32 + q / (BM / 4), r4 = (q % (BM / 4)) * 4;
      if (r4 >= rows || c >= cols) continue;
      och_f32x4 v = *reinterpret_cast<const och_f32x4 *>(shares + (size_t)c * BM + r4);
      for (uint32_t t = 1; t < p.split; t++)
      {  const och_f32x4 w = *reinterpret_cast<const och_f32x4 *>(shares + (size_t)t * BM * BN + (size_t)c * BM + r4);
         v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
      }
      v.x *= alpha; v.y *= alpha; v.z *= alpha; v.w *= alpha;
      och_f32x4 *dst = reinterpret_cast<och_f32x4 *>(p.C + ((int64_t)(m0 + r4) + (int64_t)(n0 + c) * p.ldC) * 4);
      if (beta != 0) { const och_f32x4 old = *dst; v.x += beta * old.x; v.y += beta * old.y; v.z += beta * old.z; v.w += beta * old.w; }
      *dst = v;
   }
}

/* Into how many shares the tiles of the last round are cut (1: not at all): the round must be at most half full, every
   share at least 8 slabs long, at most 8 shares per tile (64 when the whole product is less than one round), and all shares must fit into the stream's workspace. *rounds: the rounds of the compute
   units the product then takes (for the cost model of the caller); the cut round counts as the length of a share plus
   what every block spends outside its main loop (about 6 slabs' worth) over the length of a whole tile. */
int gemm_float_pipe_split(const GemmArgs &g, int tile, double *rounds)
{
   return gemm_pipe_split_plan(g.M, g.N, g.K, (uint64_t)g.nz, g.batch.nb == 0, (uint32_t)tile, (uint32_t)tile, OCH_FP_KT, 4, (uint64_t)gemm_compute_units(), rounds);
}

/* 0: launched; 1: not a case for this kernel (the caller's other kernels take it). tile: 256 or 128; M and N multiples
   of 4, K of 32, operands aligned to 16 bytes. */
int gemm_float_pipe(const GemmArgs &g, int tile)
{
   if (g.M % 4 != 0 || g.N % 4 != 0 || g.M == 0 || g.N == 0 || g.K % OCH_FP_KT != 0 || g.K == 0 || !gemm_operands_aligned(g, 4)) return 1;
   /* a lane's offset within a slab (up to 255 columns further on) is kept in 32 bits */
   if ((int64_t)g.ldA * 4 >= (1 << 24) || (int64_t)g.ldB * 4 >= (1 << 24)) return 1;
   FloatPipeParams p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host) { memcpy(&p.alpha, g.alpha, 4); memcpy(&p.beta, g.beta, 4); }
   else { p.alpha_dev = (const float *)g.alpha; p.beta_dev = (const float *)g.beta; }
   p.batch = g.batch;
   p.tiles_m = (uint32_t)((g.M + tile - 1) / tile); p.tiles_n = (uint32_t)((g.N + tile - 1) / tile);
   uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   if (tile != 256 && tile != 128 && tile != 64) return 1;
   const int shares = gemm_float_pipe_split(g, tile, nullptr);
   uint32_t cut_tiles = 0;
   if (shares > 1)
   {  char *ws;
      if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
      cut_tiles = (uint32_t)(blocks % (uint64_t)gemm_compute_units());
      p.split = (uint32_t)shares; p.split_first = (uint32_t)blocks - cut_tiles; p.partial = reinterpret_cast<float *>(ws);
      blocks += (uint64_t)cut_tiles * (shares - 1);
   }
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   /* a K of one or two slabs on the small tile: one slab buffer and four blocks per compute unit instead of two buffers and
      two blocks (8192 x 8192 x 64: 67-74 -> 78-80 TFLOP/s; from four slabs on the two buffers win). Same MFMAs in the
      same order: the same bits. */
   const bool single = tile == 128 && shares == 1 && g.K / OCH_FP_KT <= 2;
   const dim3 grid((unsigned)blocks, 1, g.nz), block(OCH_FP_THREADS);
#define OCH_FP_LAUNCH(AK, BK, TS, SINGLE, NB)                                                                         \
   do { auto kernel = gemm_float_pipe_kernel<AK, BK, TS, SINGLE, NB>;                                                 \
        const size_t lds = ((SINGLE) ? 2 : 2 * (NB)) * (size_t)FloatSlab<AK, 64 * TS>::OPERAND;                       \
        OCH_CHECK_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kernel, grid, block, lds, g.stream, p); } while (0)
#define OCH_FP_PICK(AK, BK) do { if (tile == 256) OCH_FP_LAUNCH(AK, BK, 4, false, 2); else if (tile == 64) OCH_FP_LAUNCH(AK, BK, 1, false, 2); else if (single) OCH_FP_LAUNCH(AK, BK, 2, true, 2); else OCH_FP_LAUNCH(AK, BK, 2, false, 2); } while (0)
   if (!akc && !bkc) OCH_FP_PICK(false, false);
   else if (!akc)    OCH_FP_PICK(false, true);
   else if (!bkc)    OCH_FP_PICK(true, false);
   else              OCH_FP_PICK(true, true);
#undef OCH_FP_PICK
#undef OCH_FP_LAUNCH
   if (shares > 1)
   {  if (tile == 256) hipLaunchKernelGGL(gemm_float_pipe_finish_kernel<4>, dim3(cut_tiles, 8), dim3(256), 0, g.stream, p);
      else if (tile == 128) hipLaunchKernelGGL(gemm_float_pipe_finish_kernel<2>, dim3(cut_tiles, 4), dim3(256), 0, g.stream, p);
      else             hipLaunchKernelGGL(gemm_float_pipe_finish_kernel<1>, dim3(cut_tiles, 2), dim3(256), 0, g.stream, p);
   }
   OCH_CHECK_LAUNCH();
   return 0;
}

} /* namespace och */
