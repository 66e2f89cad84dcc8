/* double GEMM on tiles of 256 x 128 for aligned operands with M and N multiples of 2 and K of 16: C <- alpha * op(A) * op(B) + beta * C, column-major.
 *
 * The counterpart of cublasDgemm in the reference (src/core/gpu/op/tensor_blas_gpu.c:183-197). Four waves per block,
 * one per SIMD, each owning 128 x 64 of the tile as 8 x 4 tiles of v_mfma_f64_16x16x4_f64 (256 accumulator registers).
 * As in the float kernel (och_gemm_f32p.hip) the main loop holds MFMAs, LDS reads, scalar instructions and loads that go
 * from memory straight to LDS, and nothing else: a vector-ALU instruction would take its cycles away from the matrix cores.
 *
 *   - a slab is 16 k; three slab buffers of 50 KB rotate. An operand that is contiguous along k in memory lies in LDS as
 *     16-byte chunks of 2 k, chunk-major: [chunk][row][2 doubles]; lane l of a load instruction fetches one chunk of row l
 *     of 64 rows. An operand that is contiguous along m / n lies in LDS as it lies in memory, [k][rows]; a load instruction
 *     fetches one k of 128 rows. Either way the 64 lanes of a load write 1 KB of consecutive LDS.
 *   - an MFMA step consumes one double per lane and operand, lanes 16 g .. 16 g + 15 holding k-group g of four. One
 *     16-byte fragment read yields, for a k-contiguous operand, the values of one 16-row tile for two steps; for the other
 *     kind, the values of two tiles for one step, the tiles then being made of every second row (tiles 2 x and 2 x + 1 =
 *     rows 32 x + 2 r and 32 x + 2 r + 1), which is undone when C is written. Two steps are a "pair"; in step t of pair P
 *     the lanes hold k = 8 P + 2 g + t for both operands.
 *   - a pair is 64 MFMAs = 32 chunks of two, each closed by a scheduling fence; the 12 fragment reads of the NEXT pair go
 *     to the even chunks (two sets of fragment registers). The one barrier of a slab stands in front of its second pair,
 *     behind a wait for the wave's own loads of the next slab: after it slab s + 1 is complete (the second pair reads its
 *     first fragments) and nobody reads this slab's buffer again, so the second pair and the first pair of the next slab
 *     issue the 12 loads of slab s + 3 into it. A load has two slabs (16000 cycles) to arrive.
 *   - the loop body has no branches: slab numbers past the end are clamped (the last slab is loaded again into a buffer
 *     nobody reads); it is written out three times so that all LDS offsets are immediates.
 *   - C leaves through LDS in passes of 32 columns, so that memory sees 16-byte accesses along the columns of C.
 *   - accumulators, fragment reads and MFMAs are written as instructions with their registers spelled out (see below):
 *     the compiler's own placement of 32 accumulator tiles and 24 fragments costs hundreds of register moves per slab.
 */
#include "och_gemm.h"
#include "och_gemm_f64p_slab.h"
#pragma clang diagnostic ignored "-Winline-asm"

namespace och {


#define OCH_DP_BM 256
#define OCH_DP_BN 128
#define OCH_DP_THREADS 256
#define OCH_DP_A 33792                       /* LDS bytes of A's slab (256 rows), either layout */
#define OCH_DP_B 17408                       /* LDS bytes of B's slab (128 rows) */
#define OCH_DP_BUFFER (OCH_DP_A + OCH_DP_B)
#define OCH_DP_BUFFERS 3

struct DoublePipeParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   double   alpha, beta;
   const double *alpha_dev, *beta_dev;
   uint32_t tiles_m, tiles_n;
   /* the tiles of the last, partly filled round of the compute units are cut along K: tiles from split_first on are
      computed by `split` blocks each, block q of them (counted from the first such block) leaving the raw sums of its
      share of the slabs in partial[q] (a dense tile, column-major); gemm_double_pipe_finish_kernel adds the shares in
      order and applies alpha / beta. split <= 1: no tile is cut. Only without a batch. */
   uint32_t split_first, split;
   double  *partial;
   GemmBatch batch;
};

static_assert(8 * DoubleSlab<true, 256>::PLANE <= OCH_DP_A && 16 * DoubleSlab<false, 256>::ROWP <= OCH_DP_A, "A's slab does not fit");
static_assert(8 * DoubleSlab<true, 128>::PLANE <= OCH_DP_B && 16 * DoubleSlab<false, 128>::ROWP <= OCH_DP_B, "B's slab does not fit");

/* 16 bytes of LDS into two ordinary registers pairs. Written as an instruction of its own so that the value lands in the
   ordinary registers (left to itself the compiler reads fragments into accumulation registers and copies them on every
   use). The compiler does not know that the value arrives later: every pair of steps opens with a wait for all LDS reads. */
static __device__ __forceinline__ och_f64x2 lds_read(uint32_t address, int offset)
{
   och_f64x2 v;
   asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(address), "i"(offset));
   return v;
}

/* The 32 accumulator tiles live in the accumulation registers a[0:255], tile (i, j) in a[8 (4 i + j) : 8 (4 i + j) + 7],
   addressed by name from instructions written out here: given them as values, the register allocator spreads tiles and
   fragments over both register files and spends the loop moving them. The compiler knows of the registers through the
   clobber of the zeroing below, and has no use of its own for them (everything else in this kernel lives in ordinary
   registers). It sees no MFMA either, so the waits it would add between an MFMA and a reader of its result are written
   out where such a reader follows (after the loop). */
static __device__ __forceinline__ void acc_zero()
{
   asm volatile(".set och_acc, 0\n\t.rept 256\n\tv_accvgpr_write_b32 a[och_acc], 0\n\t.set och_acc, och_acc + 1\n\t.endr" : : : "a255");
}
static __device__ __forceinline__ void acc_zero_half()                                 /* the 16 tiles of the small kernel */
{
   asm volatile(".set och_acc, 0\n\t.rept 128\n\tv_accvgpr_write_b32 a[och_acc], 0\n\t.set och_acc, och_acc + 1\n\t.endr" : : : "a127");
}
static __device__ __forceinline__ void mfma_f64(int tile, double a, double b)         /* tile += a b */
{
   asm volatile("v_mfma_f64_16x16x4_f64 a[%2:%2+7], %0, %1, a[%2:%2+7]" : : "v"(a), "v"(b), "i"(8 * tile));
}
static __device__ __forceinline__ double acc_read(int tile, int r)                     /* register r (0 .. 3) of a tile */
{
   uint32_t lo, hi;
   asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_accvgpr_read_b32 %1, a[%2+1]" : "=v"(lo), "=v"(hi) : "i"(8 * tile + 2 * r));
   return __hiloint2double((int)hi, (int)lo);
}

template <bool AKC, bool BKC>
__global__ __launch_bounds__(OCH_DP_THREADS) void gemm_double_pipe_kernel(const DoublePipeParams p)
{
   constexpr int T = 16, BM = OCH_DP_BM, BN = OCH_DP_BN, KT = OCH_DP_KT, TMS = 8, TNS = 4, WM = 128, WN = 64, THREADS = OCH_DP_THREADS;
   constexpr uint32_t OPA = OCH_DP_A, BUF = OCH_DP_BUFFER;
   typedef DoubleSlab<AKC, BM> LA;
   typedef DoubleSlab<BKC, BN> LB;
   static_assert(LA::LOADS == 8 && LB::LOADS == 4 && LA::TILES == TMS && LB::TILES == TNS, "the schedule below is written for these");
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

   acc_zero();

   /* this block's slabs: slab0 .. last of the product's K / KT (all of them unless the tile is cut) */
   const uint32_t per_share = (p.K / KT + shares - 1) / shares, slab0 = share * per_share;
   const uint32_t nslabs = slab0 + per_share <= p.K / KT ? per_share : p.K / KT - slab0, last = slab0 + nslabs - 1;
   const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)lds;      /* where the array starts in LDS */
   const uint32_t rowsA = p.M - m0 < (uint32_t)BM ? p.M - m0 : (uint32_t)BM, rowsB = p.N - n0 < (uint32_t)BN ? p.N - n0 : (uint32_t)BN;    /* of this tile */
   uint32_t offA[8], offB[4], tgtA[8], tgtB[4];
#pragma unroll
   for (int j = 0; j < 8; j++) { offA[j] = LA::load_offset(j, wave, lane, p.ldA, rowsA); tgtA[j] = lds0 + LA::load_target(j, wave); }
#pragma unroll
   for (int j = 0; j < 4; j++) { offB[j] = LB::load_offset(j, wave, lane, p.ldB, rowsB); tgtB[j] = lds0 + OPA + LB::load_target(j, wave); }
   /* the lane's read addresses in the three buffers, in registers of their own (the empty asm keeps the compiler from
      deriving one from the other with an addition at every read: the distance is beyond a read's immediate) */
   uint32_t readA[3], readB[3];
#pragma unroll
   for (int b = 0; b < 3; b++)
   {  readA[b] = lds0 + LA::read_lane(wm, lane) + b * BUF; readB[b] = lds0 + OPA + LB::read_lane(wn, lane) + b * BUF;
      asm volatile("" : "+v"(readA[b]), "+v"(readB[b]));
   }
   och_f64x2 fa[2][TMS], fb[2][TNS];

   /* load number e (0 .. 11; A's eight first) of a slab into buffer `buf` */
#define OCH_LOAD(e, baseA, baseB, buf)                                                                                 \
   do { if ((e) < 8) load_to_lds(baseA, offA[(e) % 8], tgtA[(e) % 8] + (buf) * BUF);                                   \
        else         load_to_lds(baseB, offB[(e) % 4], tgtB[(e) % 4] + (buf) * BUF); } while (0)
   /* one pair: chunk c reads fragment c / 2 of pair PN from buffer RB into set NXT when c is even and below 24, issues
      load LOAD0 + c / 6 into buffer LBUF when c % 6 == 1 and LOADS is set, then runs its two MFMAs */
#define OCH_PAIR(CUR, NXT, RB, PN, LOADS, LOAD0, LBUF)                                                                 \
   do { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                            \
        _Pragma("unroll") for (int c = 0; c < 32; c++)                                                                \
        {  if (c % 2 == 0 && c < 24)                                                                                   \
           {  if (c / 2 < TMS) fa[NXT][c / 2 % TMS] = lds_read(readA[RB], LA::read_offset(c / 2 % TMS, PN));            \
              else             fb[NXT][c / 2 % TNS] = lds_read(readB[RB], LB::read_offset(c / 2 % TNS, PN));            \
           }                                                                                                           \
           if (LOADS && c % 6 == 1) OCH_LOAD(LOAD0 + c / 6, nextA, nextB, LBUF);                                       \
           {  const int st = c / 16, m = (c % 16) * 2, i = m / TNS, j = m % TNS;                                       \
              mfma_f64(i * TNS + j, LA::value(fa[CUR], i, st), LB::value(fb[CUR], j, st));                               \
              mfma_f64(i * TNS + j + 1, LA::value(fa[CUR], i, st), LB::value(fb[CUR], j + 1, st));                       \
           }                                                                                                           \
           __builtin_amdgcn_sched_barrier(0);                                                                          \
        } } while (0)
   /* slab s in buffer CB: its first pair carries the second half of the loads of slab s + 2, its second pair the first
      half of the loads of slab s + 3 (into this buffer); at the barrier only the loads of slab s + 2 may still be under way */
#define OCH_SLAB(s, CB)                                                                                                \
   do { {  const uint32_t s2 = (slab0 + (s) + 2 < last) ? slab0 + (s) + 2 : last;                                                      \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);  \
           OCH_PAIR(0, 1, CB, 1, true, 6, (CB + 2) % 3);                                                               \
        }                                                                                                              \
        asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");                                                   \
        __syncthreads();                                                                                               \
        {  const uint32_t s3 = (slab0 + (s) + 3 < last) ? slab0 + (s) + 3 : last;                                                      \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s3 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s3 * KT);  \
           OCH_PAIR(1, 0, (CB + 1) % 3, 0, true, 0, CB);                                                               \
        } } while (0)

   {  /* slabs 0 and 1 and the first half of slab 2 */
      const uint32_t s1 = (slab0 + 1 < last) ? slab0 + 1 : last, s2 = (slab0 + 2 < last) ? slab0 + 2 : last;
      const char *nextA = LA::slab_base(pA, p.ldA, m0, slab0 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, slab0 * KT);
#pragma unroll
      for (int e = 0; e < 12; e++) OCH_LOAD(e, nextA, nextB, 0);
      nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT); nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);
#pragma unroll
      for (int e = 0; e < 12; e++) OCH_LOAD(e, nextA, nextB, 1);
      nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT); nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);
#pragma unroll
      for (int e = 0; e < 6; e++) OCH_LOAD(e, nextA, nextB, 2);
      asm volatile("s_waitcnt vmcnt(18) lgkmcnt(0)" ::: "memory");
      __syncthreads();
#pragma unroll
      for (int x = 0; x < TMS; x++) fa[0][x] = lds_read(readA[0], LA::read_offset(x, 0));
#pragma unroll
      for (int x = 0; x < TNS; x++) fb[0][x] = lds_read(readB[0], LB::read_offset(x, 0));
   }
   asm volatile("s_nop 7");                 /* the zeroed accumulators are in place */
   uint32_t s = 0;
   for (; s + 2 < nslabs; s += 3)
   {  OCH_SLAB(s, 0);
      OCH_SLAB(s + 1, 1);
      OCH_SLAB(s + 2, 2);
   }
   if (s < nslabs) OCH_SLAB(s, 0);
   if (s + 1 < nslabs) OCH_SLAB(s + 1, 1);
   asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0)" ::: "memory");       /* the last MFMAs have left the pipeline; the last loads have landed */
   __syncthreads();
#undef OCH_SLAB
#undef OCH_PAIR
#undef OCH_LOAD

   /* epilogue: accumulator register r of lane l is row-in-tile 4 r + l / 16 of A's tile and row-in-tile l % 16 of B's.
      The scaled tile goes through LDS, 32 columns at a time with a pitch of BM + 2 doubles, and leaves (after beta * C
      has been added) in 16-byte pieces that follow the columns of C. */
   double alpha = p.alpha, beta = p.beta;
   if (p.alpha_dev) alpha = *reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha);
   if (p.beta_dev)  beta = *reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);
   /* a share of a cut tile leaves its raw sums, the whole tile, in the workspace */
   char *out = pC + ((int64_t)m0 + (int64_t)n0 * p.ldC) * 8;
   int64_t ldOut = p.ldC;
   uint32_t rowsOut = rowsA, colsOut = rowsB;
   if (shares > 1)
   {  alpha = 1.0; beta = 0.0;
      out = reinterpret_cast<char *>(p.partial + (size_t)cut * BM * BN); ldOut = BM; rowsOut = BM; colsOut = BN;
   }
   constexpr int CP = BM + 2, CPASS = 32, PASSES = BN / CPASS;
   static_assert(CPASS * CP * 8 <= OCH_DP_BUFFERS * BUF, "a pass of the staged tile does not fit into the slab buffers");
   double *stage = reinterpret_cast<double *>(lds);
   for (int h = 0; h < PASSES; h++)
   {
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {  const uint32_t col = wn + LB::row(j, lane % T);
         if (col / CPASS != (uint32_t)h) continue;
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int r = 0; r < 4; r++)
               stage[(col - h * CPASS) * CP + wm + LA::row(i, 4 * r + (lane >> 4))] = alpha * acc_read(i * TNS + j, r);
      }
      __syncthreads();
      for (uint32_t q = threadIdx.x; q < CPASS * (BM / 2); q += THREADS)
      {  const uint32_t c = q / (BM / 2), r2 = (q % (BM / 2)) * 2;
         if (r2 >= rowsOut || h * CPASS + c >= colsOut) continue;      /* outside C */
         och_f64x2 v = *reinterpret_cast<const och_f64x2 *>(stage + c * CP + r2);
         och_f64x2 *dst = reinterpret_cast<och_f64x2 *>(out + ((int64_t)r2 + (int64_t)(h * CPASS + c) * ldOut) * 8);
         if (beta != 0) { const och_f64x2 old = *dst; v.x += beta * old.x; v.y += beta * old.y; }
         *dst = v;
      }
      __syncthreads();
   }
}

/* The same on tiles of 128 x 128 for products with too few tiles of 256 x 128: four waves of 64 x 64 (4 x 4 tiles, 128
   accumulation registers), two slab buffers of 34 KB, so that two blocks share a compute unit and fill each other's
   waits. Slab s in buffer s % 2: its first pair carries the second half of the 8 loads of slab s + 1 (into the other
   buffer), the barrier behind a wait for all loads stands in front of its second pair, which reads the first fragments
   of slab s + 1 and carries the first half of the loads of slab s + 2 (into this buffer). */
template <bool AKC, bool BKC>
__global__ __launch_bounds__(OCH_DP_THREADS, 2) void gemm_double_pipe_small_kernel(const DoublePipeParams p)
{
   constexpr int T = 16, BM = 128, BN = 128, KT = OCH_DP_KT, TMS = 4, TNS = 4, WM = 64, WN = 64, THREADS = OCH_DP_THREADS;
   constexpr uint32_t OPA = OCH_DP_B, BUF = 2 * OCH_DP_B;
   typedef DoubleSlab<AKC, BM> LA;
   typedef DoubleSlab<BKC, BN> LB;
   static_assert(LA::LOADS == 4 && LB::LOADS == 4 && LA::TILES == TMS && LB::TILES == TNS, "the schedule below is written for these");
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

   acc_zero_half();

   /* this block's slabs: slab0 .. last of the product's K / KT (all of them unless the tile is cut) */
   const uint32_t per_share = (p.K / KT + shares - 1) / shares, slab0 = share * per_share;
   const uint32_t nslabs = slab0 + per_share <= p.K / KT ? per_share : p.K / KT - slab0, last = slab0 + nslabs - 1;
   const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)lds;      /* where the array starts in LDS */
   const uint32_t rowsA = p.M - m0 < (uint32_t)BM ? p.M - m0 : (uint32_t)BM, rowsB = p.N - n0 < (uint32_t)BN ? p.N - n0 : (uint32_t)BN;    /* of this tile */
   uint32_t offA[4], offB[4], tgtA[4], tgtB[4];
#pragma unroll
   for (int j = 0; j < 4; j++)
   {  offA[j] = LA::load_offset(j, wave, lane, p.ldA, rowsA); tgtA[j] = lds0 + LA::load_target(j, wave);
      offB[j] = LB::load_offset(j, wave, lane, p.ldB, rowsB); tgtB[j] = lds0 + OPA + LB::load_target(j, wave);
   }
   uint32_t readA[2], readB[2];
#pragma unroll
   for (int b = 0; b < 2; b++)
   {  readA[b] = lds0 + LA::read_lane(wm, lane) + b * BUF; readB[b] = lds0 + OPA + LB::read_lane(wn, lane) + b * BUF;
      asm volatile("" : "+v"(readA[b]), "+v"(readB[b]));
   }
   och_f64x2 fa[2][TMS], fb[2][TNS];

#define OCH_LOAD(e, baseA, baseB, buf)                                                                                 \
   do { if ((e) < 4) load_to_lds(baseA, offA[(e) % 4], tgtA[(e) % 4] + (buf) * BUF);                                   \
        else         load_to_lds(baseB, offB[(e) % 4], tgtB[(e) % 4] + (buf) * BUF); } while (0)
   /* one pair of steps = 32 MFMAs = 16 chunks: chunk c reads fragment c / 2 of pair PN from buffer RB into set NXT when c
      is even, issues load LOAD0 + c / 4 into buffer LBUF when c % 4 == 2, then runs its two MFMAs */
#define OCH_PAIR(CUR, NXT, RB, PN, LOAD0, LBUF)                                                                        \
   do { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                            \
        _Pragma("unroll") for (int c = 0; c < 16; c++)                                                                \
        {  if (c % 2 == 0)                                                                                             \
           {  if (c / 2 < TMS) fa[NXT][c / 2 % TMS] = lds_read(readA[RB], LA::read_offset(c / 2 % TMS, PN));            \
              else             fb[NXT][c / 2 % TNS] = lds_read(readB[RB], LB::read_offset(c / 2 % TNS, PN));            \
           }                                                                                                           \
           if (c % 4 == 2) OCH_LOAD(LOAD0 + c / 4, nextA, nextB, LBUF);                                                \
           {  const int st = c / 8, m = (c % 8) * 2, i = m / TNS, j = m % TNS;                                         \
              mfma_f64(i * TNS + j, LA::value(fa[CUR], i, st), LB::value(fb[CUR], j, st));                             \
              mfma_f64(i * TNS + j + 1, LA::value(fa[CUR], i, st), LB::value(fb[CUR], j + 1, st));                     \
           }                                                                                                           \
           __builtin_amdgcn_sched_barrier(0);                                                                          \
        } } while (0)
#define OCH_SLAB(s, CB)                                                                                                \
   do { {  const uint32_t s1 = (slab0 + (s) + 1 < last) ? slab0 + (s) + 1 : last;                                                      \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);  \
           OCH_PAIR(0, 1, CB, 1, 4, 1 - CB);                                                                           \
        }                                                                                                              \
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                                                    \
        __syncthreads();                                                                                               \
        {  const uint32_t s2 = (slab0 + (s) + 2 < last) ? slab0 + (s) + 2 : last;                                                      \
           const char *nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);  \
           OCH_PAIR(1, 0, 1 - CB, 0, 0, CB);                                                                           \
        } } while (0)

   {  /* slab 0 and the first half of slab 1 */
      const uint32_t s1 = (slab0 + 1 < last) ? slab0 + 1 : last;
      const char *nextA = LA::slab_base(pA, p.ldA, m0, slab0 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, slab0 * KT);
#pragma unroll
      for (int e = 0; e < 8; e++) OCH_LOAD(e, nextA, nextB, 0);
      nextA = LA::slab_base(pA, p.ldA, m0, s1 * KT); nextB = LB::slab_base(pB, p.ldB, n0, s1 * KT);
#pragma unroll
      for (int e = 0; e < 4; e++) OCH_LOAD(e, nextA, nextB, 1);
      asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
      __syncthreads();
#pragma unroll
      for (int x = 0; x < TMS; x++) fa[0][x] = lds_read(readA[0], LA::read_offset(x, 0));
#pragma unroll
      for (int x = 0; x < TNS; x++) fb[0][x] = lds_read(readB[0], LB::read_offset(x, 0));
   }
   asm volatile("s_nop 7");                 /* the zeroed accumulators are in place */
   uint32_t s = 0;
   for (; s + 1 < nslabs; s += 2)
   {  OCH_SLAB(s, 0);
      OCH_SLAB(s + 1, 1);
   }
   if (s < nslabs) OCH_SLAB(s, 0);
   asm volatile("s_nop 15\n\ts_nop 15\n\ts_waitcnt vmcnt(0)" ::: "memory");       /* the last MFMAs have left the pipeline; the last loads have landed */
   __syncthreads();
#undef OCH_SLAB
#undef OCH_PAIR
#undef OCH_LOAD

   double alpha = p.alpha, beta = p.beta;
   if (p.alpha_dev) alpha = *reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha);
   if (p.beta_dev)  beta = *reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);
   /* a share of a cut tile leaves its raw sums, the whole tile, in the workspace */
   char *out = pC + ((int64_t)m0 + (int64_t)n0 * p.ldC) * 8;
   int64_t ldOut = p.ldC;
   uint32_t rowsOut = rowsA, colsOut = rowsB;
   if (shares > 1)
   {  alpha = 1.0; beta = 0.0;
      out = reinterpret_cast<char *>(p.partial + (size_t)cut * BM * BN); ldOut = BM; rowsOut = BM; colsOut = BN;
   }
   constexpr int CP = BM + 2, CPASS = 32, PASSES = BN / CPASS;
   static_assert(CPASS * CP * 8 <= 2 * BUF, "a pass of the staged tile does not fit into the slab buffers");
   double *stage = reinterpret_cast<double *>(lds);
   for (int h = 0; h < PASSES; h++)
   {
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {  const uint32_t col = wn + LB::row(j, lane % T);
         if (col / CPASS != (uint32_t)h) continue;
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int r = 0; r < 4; r++)
               stage[(col - h * CPASS) * CP + wm + LA::row(i, 4 * r + (lane >> 4))] = alpha * acc_read(i * TNS + j, r);
      }
      __syncthreads();
      for (uint32_t q = threadIdx.x; q < CPASS * (BM / 2); q += THREADS)
      {  const uint32_t c = q / (BM / 2), r2 = (q % (BM / 2)) * 2;
         if (r2 >= rowsOut || h * CPASS + c >= colsOut) continue;      /* outside C */
         och_f64x2 v = *reinterpret_cast<const och_f64x2 *>(stage + c * CP + r2);
         och_f64x2 *dst = reinterpret_cast<och_f64x2 *>(out + ((int64_t)r2 + (int64_t)(h * CPASS + c) * ldOut) * 8);
         if (beta != 0) { const och_f64x2 old = *dst; v.x += beta * old.x; v.y += beta * old.y; }
         *dst = v;
      }
      __syncthreads();
   }
}

/* The shares of the cut tiles, added in the order of their slabs, times alpha, plus beta * C: a block per 16 columns of a
   cut tile (grid y), 16 bytes of a column of C per thread and trip. */
template <int BM>
__global__ __launch_bounds__(256) void gemm_double_pipe_finish_kernel(const DoublePipeParams p)
{
   constexpr uint32_t BN = 128;
   const uint32_t tile = p.split_first + blockIdx.x, tile_m = tile % p.tiles_m, tile_n = tile / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const uint32_t rows = p.M - m0 < (uint32_t)BM ? p.M - m0 : (uint32_t)BM, cols = p.N - n0 < BN ? p.N - n0 : BN;
   const double alpha = p.alpha_dev ? *p.alpha_dev : p.alpha, beta = p.beta_dev ? *p.beta_dev : p.beta;
   const double *shares = p.partial + (size_t)blockIdx.x * p.split * BM * BN;
   for (uint32_t q = threadIdx.x; q < 16 * (BM / 2); q += 256)
   {  const uint32_t c = blockIdx.y * 16 + q / (BM / 2), r2 = (q % (BM / 2)) * 2;
      if (r2 >= rows || c >= cols) continue;
      och_f64x2 v = *reinterpret_cast<const och_f64x2 *>(shares + (size_t)c * BM + r2);
      for (uint32_t t = 1; t < p.split; t++)
      {  const och_f64x2 w = *reinterpret_cast<const och_f64x2 *>(shares + (size_t)t * BM * BN + (size_t)c * BM + r2);
         v.x += w.x; v.y += w.y;
      }
      v.x *= alpha; v.y *= alpha;
      och_f64x2 *dst = reinterpret_cast<och_f64x2 *>(p.C + ((int64_t)(m0 + r2) + (int64_t)(n0 + c) * p.ldC) * 8);
      if (beta != 0) { const och_f64x2 old = *dst; v.x += beta * old.x; v.y += beta * old.y; }
      *dst = v;
   }
}

/* Into how many shares the tiles of the last round are cut (1: not at all): the round must be at most half full, every
   share at least 8 slabs long, at most 8 shares per tile (64 when the whole product is less than one round), and all shares must fit into the stream's workspace. *rounds: the rounds of the compute
   units the product then takes (for the cost model of the caller); the cut round counts as the length of a share plus
   what every block spends outside its main loop (about 6 slabs' worth) over the length of a whole tile. */
int gemm_double_pipe_split(const GemmArgs &g, int tile_m, double *rounds)
{
   return gemm_pipe_split_plan(g.M, g.N, g.K, (uint64_t)g.nz, g.batch.nb == 0, (uint32_t)tile_m, OCH_DP_BN, OCH_DP_KT, 8, (uint64_t)gemm_compute_units(), rounds);
}

/* 0: launched; 1: not a case for this kernel (the caller's other kernels take it): M and N multiples of 2, K of 16,
   operands aligned to 16 bytes */
int gemm_double_pipe(const GemmArgs &g, int tile_m)          /* tile_m: 256 (tiles of 256 x 128) or 128 (tiles of 128 x 128) */
{
   if (g.M % 2 != 0 || g.N % 2 != 0 || g.M == 0 || g.N == 0 || g.K % OCH_DP_KT != 0 || g.K == 0 || !gemm_operands_aligned(g, 8)) return 1;
   /* a lane's offset within a slab (up to 255 columns further on) is kept in 32 bits */
   if ((int64_t)g.ldA * 8 >= (1 << 24) || (int64_t)g.ldB * 8 >= (1 << 24)) return 1;
   DoublePipeParams p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host) { memcpy(&p.alpha, g.alpha, 8); memcpy(&p.beta, g.beta, 8); }
   else { p.alpha_dev = (const double *)g.alpha; p.beta_dev = (const double *)g.beta; }
   p.batch = g.batch;
   if (tile_m != 256 && tile_m != 128) return 1;
   p.tiles_m = (uint32_t)((g.M + tile_m - 1) / tile_m); p.tiles_n = (uint32_t)((g.N + OCH_DP_BN - 1) / OCH_DP_BN);
   uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   const int shares = gemm_double_pipe_split(g, tile_m, nullptr);
   uint32_t cut_tiles = 0;
   if (shares > 1)
   {  char *ws;
      if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
      cut_tiles = (uint32_t)(blocks % (uint64_t)gemm_compute_units());
      p.split = (uint32_t)shares; p.split_first = (uint32_t)blocks - cut_tiles; p.partial = reinterpret_cast<double *>(ws);
      blocks += (uint64_t)cut_tiles * (shares - 1);
   }
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   const dim3 grid((unsigned)blocks, 1, g.nz), block(OCH_DP_THREADS);
   const size_t lds = tile_m == 256 ? OCH_DP_BUFFERS * (size_t)OCH_DP_BUFFER : 4 * (size_t)OCH_DP_B;
#define OCH_DP_LAUNCH(AK, BK)                                                                                         \
   do { auto kernel = tile_m == 256 ? gemm_double_pipe_kernel<AK, BK> : gemm_double_pipe_small_kernel<AK, BK>;        \
        OCH_CHECK_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kernel, grid, block, lds, g.stream, p); } while (0)
   if (!akc && !bkc) OCH_DP_LAUNCH(false, false);
   else if (!akc)    OCH_DP_LAUNCH(false, true);
   else if (!bkc)    OCH_DP_LAUNCH(true, false);
   else              OCH_DP_LAUNCH(true, true);
#undef OCH_DP_LAUNCH
   if (shares > 1)
   {  if (tile_m == 256) hipLaunchKernelGGL(gemm_double_pipe_finish_kernel<256>, dim3(cut_tiles, 8), dim3(256), 0, g.stream, p);
      else               hipLaunchKernelGGL(gemm_double_pipe_finish_kernel<128>, dim3(cut_tiles, 8), dim3(256), 0, g.stream, p);
   }
   OCH_CHECK_LAUNCH();
   return 0;
}

} /* namespace och */
