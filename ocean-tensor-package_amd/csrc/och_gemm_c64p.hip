/* complex double GEMM on tiles of 128 x 64 for 16-byte aligned operands and K a multiple of 16:
 * C <- alpha * op(A) * op(B) + beta * C, column-major, op = none, transposition or conjugate transposition.
 *
 * The counterpart of cublasZgemm in the reference (src/core/gpu/op/tensor_blas_gpu.c:183-197). The double kernel
 * (och_gemm_f64p.hip) with complex operands: four waves per block, one per SIMD, each owning 64 x 32 complex elements as
 * 4 x 2 tiles of 16 x 16, every tile with FOUR real accumulators -- Ar Br, Ai Bi, Ar Bi and Ai Br summed over k by
 * v_mfma_f64_16x16x4_f64 -- which are combined when C is written (the matrix cores have no operand negation; the signs of
 * the combination are all that conjugation changes). 32 accumulators of 8 registers, 32 independent MFMAs per step, the
 * 256 accumulation registers addressed by name, as in the double kernel; the main loop holds MFMAs, LDS reads, scalar
 * instructions and loads that go from memory straight to LDS, and no vector arithmetic.
 *
 *   - an element is 16 bytes, one lane's share of a load to LDS and one fragment read: a slab of 16 k lies in LDS as
 *     [k][row][re, im] whichever way the operand lies in memory; only the addresses the lanes load from differ (lane =
 *     row of 64 for one k; an operand contiguous along k then has each row's 16 k fetched by 16 instructions).
 *   - a fragment read yields (re, im) of one tile for one step; in step t the lanes 16 g .. 16 g + 15 hold k = 4 t + g.
 *   - schedule, three rotating buffers of 50 KB, barrier and clamped loads are those of the double kernel: pairs of two
 *     steps = 64 MFMAs = 32 chunks of two; 12 fragment reads of the next pair on the even chunks, 12 loads per slab.
 *   - any M and N: an element is a whole 16-byte piece of C. The last tiles clamp their loads to the rows that exist.
 */
#include "och_gemm.h"
#include "och_gemm_c64p_slab.h"
#pragma clang diagnostic ignored "-Winline-asm"

namespace och {


#define OCH_ZP_BM 128
#define OCH_ZP_BN 64
#define OCH_ZP_THREADS 256
#define OCH_ZP_A 33792                       /* LDS bytes of A's slab (128 rows of 16 k) */
#define OCH_ZP_B 17408                       /* LDS bytes of B's slab (64 rows) */
#define OCH_ZP_BUFFER (OCH_ZP_A + OCH_ZP_B)
#define OCH_ZP_BUFFERS 3

struct CDoublePipeParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   double   alpha[2], beta[2];          /* (re, im) */
   const double *alpha_dev, *beta_dev;
   int      conjA, conjB;
   uint32_t tiles_m, tiles_n;
   /* the tiles of the last, partly filled round of the compute units are cut along K: tiles from split_first on are
      computed by `split` blocks each, block q of them (counted from the first such block) leaving the raw complex sums of
      its share of the slabs in partial[q] (a dense tile, column-major); the finish kernel adds the shares in order and
      applies alpha / beta. split <= 1: no tile is cut. Only without a batch. */
   uint32_t split_first, split;
   double *partial;
   GemmBatch batch;
};

static_assert(16 * CDoubleSlab<true, 128>::PLANE <= OCH_ZP_A && 16 * CDoubleSlab<true, 64>::PLANE <= OCH_ZP_B, "the slabs do not fit");

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
__global__ __launch_bounds__(OCH_ZP_THREADS) void gemm_cdouble_pipe_kernel(const CDoublePipeParams p)
{
   constexpr int T = 16, BM = OCH_ZP_BM, BN = OCH_ZP_BN, KT = OCH_ZP_KT, TMS = 4, TNS = 2, WM = 64, WN = 32, THREADS = OCH_ZP_THREADS;
   constexpr uint32_t OPA = OCH_ZP_A, BUF = OCH_ZP_BUFFER;
   typedef CDoubleSlab<AKC, BM> LA;
   typedef CDoubleSlab<BKC, BN> LB;
   static_assert(LA::LOADS == 8 && LB::LOADS == 4 && LA::TILES == TMS && LB::TILES == TNS && LA::READS == 8 && LB::READS == 4, "the schedule below is written for these");
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
   och_f64x2 fa[2][8], fb[2][4];

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
           {  if (c / 2 < 8) fa[NXT][c / 2 % 8] = lds_read(readA[RB], LA::read_offset(c / 2 % 8, PN));                  \
              else           fb[NXT][c / 2 % 4] = lds_read(readB[RB], LB::read_offset(c / 2 % 4, PN));                  \
           }                                                                                                           \
           if (LOADS && c % 6 == 1) OCH_LOAD(LOAD0 + c / 6, nextA, nextB, LBUF);                                       \
           {  const int st = c / 16, tile = (c % 16) / 2, i = tile / TNS, j = tile % TNS, ci = c % 2;   /* A's real part, then its imaginary part */ \
              mfma_f64(4 * tile + ci, LA::value(fa[CUR], i, st, ci), LB::value(fb[CUR], j, st, ci));                    \
              mfma_f64(4 * tile + 2 + ci, LA::value(fa[CUR], i, st, ci), LB::value(fb[CUR], j, st, 1 - ci));            \
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
      for (int x = 0; x < 8; x++) fa[0][x] = lds_read(readA[0], LA::read_offset(x, 0));
#pragma unroll
      for (int x = 0; x < 4; x++) fb[0][x] = lds_read(readB[0], LB::read_offset(x, 0));
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
      Tile t keeps Ar Br, Ai Bi, Ar Bi, Ai Br in accumulators 4 t .. 4 t + 3: real part Ar Br -+ Ai Bi, imaginary part
      +- Ar Bi +- Ai Br, the signs by the conjugations. The scaled tile goes through LDS, 16 columns at a time with a pitch
      of BM + 1 elements, and leaves (after beta * C has been added) element by element, 16 bytes each, along the columns of C. */
   double ar = p.alpha[0], ai = p.alpha[1], br = p.beta[0], bi = p.beta[1];
   if (p.alpha_dev) { const double *q = reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha); ar = q[0]; ai = q[1]; }
   if (p.beta_dev)  { const double *q = reinterpret_cast<const double *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta); br = q[0]; bi = q[1]; }
   const double sq = (p.conjA != p.conjB) ? 1.0 : -1.0, s1 = p.conjB ? -1.0 : 1.0, s2 = p.conjA ? -1.0 : 1.0;
   /* a share of a cut tile leaves its raw sums, the whole tile, in the workspace */
   char *out = pC + ((int64_t)m0 + (int64_t)n0 * p.ldC) * 16;
   int64_t ldOut = p.ldC;
   uint32_t rowsOut = rowsA, colsOut = rowsB;
   if (shares > 1)
   {  ar = 1; ai = 0; br = 0; bi = 0;
      out = reinterpret_cast<char *>(p.partial + (size_t)cut * BM * BN * 2); ldOut = BM; rowsOut = BM; colsOut = BN;
   }
   constexpr int CP = BM + 1, CPASS = 16, PASSES = BN / CPASS;
   static_assert(CPASS * CP * 16 <= OCH_ZP_BUFFERS * BUF, "a pass of the staged tile does not fit into the slab buffers");
   och_f64x2 *stage = reinterpret_cast<och_f64x2 *>(lds);
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
            {  const int tile = i * TNS + j;
               const double cr = acc_read(4 * tile, r) + sq * acc_read(4 * tile + 1, r), ci = s1 * acc_read(4 * tile + 2, r) + s2 * acc_read(4 * tile + 3, r);
               stage[(col - h * CPASS) * CP + wm + LA::row(i, 4 * r + (lane >> 4))] = och_f64x2{ar * cr - ai * ci, ar * ci + ai * cr};
            }
      }
      __syncthreads();
      for (uint32_t q = threadIdx.x; q < CPASS * BM; q += THREADS)
      {  const uint32_t c = q / BM, r1 = q % BM;
         if (r1 >= rowsOut || h * CPASS + c >= colsOut) continue;      /* outside C */
         och_f64x2 v = stage[c * CP + r1];
         och_f64x2 *dst = reinterpret_cast<och_f64x2 *>(out + ((int64_t)r1 + (int64_t)(h * CPASS + c) * ldOut) * 16);
         if (br != 0 || bi != 0) { const och_f64x2 old = *dst; v.x += br * old.x - bi * old.y; v.y += br * old.y + bi * old.x; }
         *dst = v;
      }
      __syncthreads();
   }
}

/* The shares of the cut tiles, added in the order of their slabs, times alpha, plus beta * C: a block per 16 columns of a
   cut tile (grid y), one element of C per thread and trip. */
__global__ __launch_bounds__(256) void gemm_cdouble_pipe_finish_kernel(const CDoublePipeParams p)
{
   constexpr uint32_t BM = 128, BN = 64;
   const uint32_t tile = p.split_first + blockIdx.x, tile_m = tile % p.tiles_m, tile_n = tile / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const uint32_t rows = p.M - m0 < BM ? p.M - m0 : BM, cols = p.N - n0 < BN ? p.N - n0 : BN;
   const double ar = p.alpha_dev ? p.alpha_dev[0] : p.alpha[0], ai = p.alpha_dev ? p.alpha_dev[1] : p.alpha[1];
   const double br = p.beta_dev ? p.beta_dev[0] : p.beta[0], bi = p.beta_dev ? p.beta_dev[1] : p.beta[1];
   const double *shares = p.partial + (size_t)blockIdx.x * p.split * BM * BN * 2;
   for (uint32_t q = threadIdx.x; q < 16 * BM; q += 256)
   {  const uint32_t c = blockIdx.y * 16 + q / BM, r = q % BM;
      if (r >= rows || c >= cols) continue;
      double sr = 0, si = 0;
      for (uint32_t t = 0; t < p.split; t++)
      {  const double *w = shares + ((size_t)t * BM * BN + (size_t)c * BM + r) * 2;
         sr += w[0]; si += w[1];
      }
      double vr = ar * sr - ai * si, vi = ar * si + ai * sr;
      double *dst = reinterpret_cast<double *>(p.C + ((int64_t)(m0 + r) + (int64_t)(n0 + c) * p.ldC) * 16);
      if (br != 0 || bi != 0) { const double cr = dst[0], ci = dst[1]; vr += br * cr - bi * ci; vi += br * ci + bi * cr; }
      dst[0] = vr; dst[1] = vi;
   }
}

/* Into how many shares the tiles of the last round are cut (1: not at all): the round must be at most half full, every
   share at least 8 slabs long, at most 8 shares per tile (64 when the whole product is less than one round), and all shares must fit into the stream's workspace. *rounds: the rounds of the compute
   units the product then takes (for the cost model of the caller); the cut round counts as the length of a share plus
   what every block spends outside its main loop (about 6 slabs' worth) over the length of a whole tile. */
int gemm_cdouble_pipe_split(const GemmArgs &g, double *rounds)
{
   return gemm_pipe_split_plan(g.M, g.N, g.K, (uint64_t)g.nz, g.batch.nb == 0, 128, 64, 16, 16, (uint64_t)gemm_compute_units(), rounds);
}

/* 0: launched; 1: not a case for this kernel (the caller's other kernel takes it): K a multiple of 16, operands aligned
   to 16 bytes (every complex double is) */
int gemm_cdouble_pipe(const GemmArgs &g)
{
   if (g.M == 0 || g.N == 0 || g.K % OCH_ZP_KT != 0 || g.K == 0 || !gemm_operands_aligned(g, 16)) return 1;
   /* a lane's offset within a slab (up to 127 columns further on) is kept in 32 bits */
   if ((int64_t)g.ldA * 16 >= (1 << 24) || (int64_t)g.ldB * 16 >= (1 << 24)) return 1;
   CDoublePipeParams p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host) { memcpy(p.alpha, g.alpha, 16); memcpy(p.beta, g.beta, 16); }
   else { p.alpha_dev = (const double *)g.alpha; p.beta_dev = (const double *)g.beta; }
   p.batch = g.batch;
   p.conjA = (g.transA == 'C'); p.conjB = (g.transB == 'C');
   p.tiles_m = (uint32_t)((g.M + OCH_ZP_BM - 1) / OCH_ZP_BM); p.tiles_n = (uint32_t)((g.N + OCH_ZP_BN - 1) / OCH_ZP_BN);
   uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   const int shares = gemm_cdouble_pipe_split(g, nullptr);
   uint32_t cut_tiles = 0;
   if (shares > 1)
   {  char *ws;
      if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
      cut_tiles = (uint32_t)(blocks % (uint64_t)gemm_compute_units());
      p.split = (uint32_t)shares; p.split_first = (uint32_t)blocks - cut_tiles; p.partial = reinterpret_cast<double *>(ws);
      blocks += (uint64_t)cut_tiles * (shares - 1);
   }
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   const dim3 grid((unsigned)blocks, 1, g.nz), block(OCH_ZP_THREADS);
   const size_t lds = OCH_ZP_BUFFERS * (size_t)OCH_ZP_BUFFER;
#define OCH_ZP_LAUNCH(AK, BK)                                                                                         \
   do { auto kernel = gemm_cdouble_pipe_kernel<AK, BK>;                                                               \
        OCH_CHECK_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kernel, grid, block, lds, g.stream, p); } while (0)
   if (!akc && !bkc) OCH_ZP_LAUNCH(false, false);
   else if (!akc)    OCH_ZP_LAUNCH(false, true);
   else if (!bkc)    OCH_ZP_LAUNCH(true, false);
   else              OCH_ZP_LAUNCH(true, true);
#undef OCH_ZP_LAUNCH
   if (shares > 1) hipLaunchKernelGGL(gemm_cdouble_pipe_finish_kernel, dim3(cut_tiles, 4), dim3(256), 0, g.stream, p);
   OCH_CHECK_LAUNCH();
   return 0;
}

} /* namespace och */
