/* Half-precision GEMM on the matrix cores: C <- alpha * op(A) * op(B) + beta * C, column-major, half in memory.
 *
 * The reference multiplies half matrices with cublasHgemm where the device has it and otherwise converts the operands to
 * float, runs the float product and converts back (src/core/interface/tensor_itf.c:6388-6400,
 * src/core/gpu/op/tensor_blas_gpu.c:259-286). Here products of halves are accumulated in float by
 * v_mfma_f32_32x32x16_f16, alpha and beta are applied in float, and the result is rounded to half once with the
 * conversion every other operation uses -- the arithmetic of the float route.
 *
 * A block of NWM x NWN waves owns a (NWM*WM) x (NWN*WN) tile of C, each wave WM x WN of it as 32 x 32 MFMA tiles. Per K
 * step of KT = 64 the block stages slabs of op(A) and op(B) through LDS, loading slab s+1 from memory into registers before the
 * MFMAs of slab s and writing it to the other LDS buffer afterwards. An MFMA operand is eight consecutive k of one row
 * (column) per lane: a k-contiguous operand lies in LDS as 16-byte chunks of 8 k and a fragment is one 16-byte LDS read.
 * An operand that is contiguous along k in memory ('T' for A, 'N' for B) arrives in that shape; one that is contiguous
 * along m / n lies in LDS as in memory, and its fragments come out of transposing LDS reads (ds_read_b64_tr_b16).
 */
#include "och_gemm.h"

namespace och {

/* The conversions of the epilogue. The library's general device conversions (och_dtypes.h) keep their rare cases behind
   wave-uniform branches, which pays in a streaming kernel; unrolled over the 256 accumulators of a wave here they cost the
   kernel its registers (a kilobyte and more of scratch per lane, and the 8192^3 product 21 ms instead of 1). So: the
   integer routine for float -> half, and the hardware converter for finite halves with the integer routine for the rest. */
static __device__ __forceinline__ float gemm_half_to_float(half_t hh)
{
   uint32_t h = hh.v;
   uint32_t s = (h & 0x8000u) << 16;
   h &= 0x7FFFu;
   if (h == 0) return 0.f;                       /* both zeros map to +0 */
   uint32_t e = h & 0x7C00u;
   if (e != 0x7C00u) { _Float16 x; __builtin_memcpy(&x, &hh.v, 2); return (float)x; }      /* exact, subnormals included */
   return bits_to_float((h << 13) | 0x7F800000u | s);                                       /* Inf, NaN with its payload */
}
static __device__ __forceinline__ half_t gemm_float_to_half(float f) { return float_to_half_soft(f); }

typedef _Float16 och_h8 __attribute__((ext_vector_type(8)));
typedef short och_i16x4 __attribute__((ext_vector_type(4)));

struct HalfGemmParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   half_t   alpha, beta;                /* when the scalars live in host memory */
   const half_t *alpha_dev, *beta_dev;  /* non-null: read the scalar from device memory */
   int      alignedA, alignedB, alignedC; /* base pointer, leading dimension and batch strides allow 128-bit accesses */
   uint32_t tiles_m, tiles_n;
   GemmBatch batch;
   /* split K (few tiles, long K; only without a batch): grid z is the slice, every slice covers split_slabs slabs of K and
      leaves its raw float sums in partial[z] (dense M x N planes); gemm_half_finish_kernel adds the slices in order */
   uint32_t split_slabs;
   float   *partial;
};

/* Moves a BMN x KT slab of an operand (2-byte elements) from memory to registers and on to LDS, 16 bytes at a time, and
   reads MFMA fragments (eight consecutive k of one row per lane) from there.
   KC (contiguous along k in memory): a thread loads one chunk of 8 k of one row; LDS holds [chunk of 8 k][row][8 halves],
   32 bytes of padding after every chunk plane; eight neighbouring lanes store the eight chunks of a row, and a fragment
   is one 16-byte read (32 neighbouring rows of one chunk plane: 512 consecutive bytes per half wave).
   !KC (contiguous along the row index): a thread loads 8 neighbouring rows of one k, for NV consecutive k, and LDS holds
   the slab as it lies in memory, [k][row] with a pitch of BMN + 16 halves. The fragments come out of transposing reads
   (ds_read_b64_tr_b16): in every group of 16 lanes, lanes 4 q .. 4 q + 3 read 16 neighbouring rows of k + q, and lane i
   of the group receives row i of k .. k + 3; two such reads make the eight k of a fragment. No register transposition,
   no permuted rows. */
template <bool KC, bool EDGE, int BMN, int KT, int THREADS>
struct HalfSlab
{
   static constexpr int NV = BMN * KT / 8 / THREADS;                   /* 16-byte loads per thread */
   static constexpr int PLANE = BMN * 8 + 16;                          /* KC: halves per chunk plane */
   static constexpr int PITCH = BMN + 16;                              /* !KC: halves from one k to the next; 32 bytes more than the rows so that the four k of a transposing read meet different banks */
   static constexpr int SIZE = KC ? (KT / 8) * PLANE : KT * PITCH;     /* halves per LDS buffer */
   static_assert(NV >= 1 && (BMN * KT) % (8 * THREADS) == 0, "slab does not divide among the threads");
   och_gu32x4 reg[NV];

   /* LDS slot -> row of the tile: the same for both layouts (kept as the one place that says so) */
   static __device__ __forceinline__ uint32_t row_of_slot(uint32_t slot) { return slot; }
   static constexpr uint32_t row_step(uint32_t o) { return o; }
   static __device__ __forceinline__ void where(int v, uint32_t &mn, uint32_t &k)
   {  if (!KC) { mn = (threadIdx.x % (BMN / 8)) * 8; k = (threadIdx.x / (BMN / 8)) * NV + v; }
      else     { const uint32_t q = threadIdx.x + THREADS * v; k = (q % (KT / 8)) * 8; mn = q / (KT / 8); }
   }
   /* element (mn, k) of op(.) lives at mn + k * ld (!KC) or k + mn * ld (KC) */
   __device__ __forceinline__ void fetch(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0, uint32_t MN, uint32_t K, int aligned)
   {
#pragma unroll
      for (int v = 0; v < NV; v++)
      {  uint32_t mn, k; where(v, mn, k);
         const int64_t gm = (int64_t)mn0 + mn, gk = (int64_t)k0 + k;
         const char *at = mat + (KC ? (gk + gm * ld) : (gm + gk * ld)) * 2;
         if (!EDGE) { reg[v] = *reinterpret_cast<const och_gu32x4 *>(at); continue; }
         /* edge tiles: a vector that lies inside the matrix (and is aligned) is still one load, one that lies outside is
            zero without touching memory; element-wise loads remain for vectors that straddle the border or are unaligned */
         const bool some = KC ? (gm < (int64_t)MN && gk < (int64_t)K) : (gk < (int64_t)K && gm < (int64_t)MN);
         const bool all  = KC ? (gm < (int64_t)MN && gk + 8 <= (int64_t)K) : (gk < (int64_t)K && gm + 8 <= (int64_t)MN);
         if (all && aligned) reg[v] = *reinterpret_cast<const och_gu32x4 *>(at);
         else
         {  uint32_t w[4] = { 0, 0, 0, 0 };
            if (some)
            {
#pragma unroll
               for (int e = 0; e < 8; e++)
               {  const bool ok = KC ? (gk + e < (int64_t)K) : (gm + e < (int64_t)MN);
                  if (ok) w[e >> 1] |= (uint32_t)*reinterpret_cast<const uint16_t *>(at + 2 * e) << (16 * (e & 1));
               }
            }
            reg[v].x = w[0]; reg[v].y = w[1]; reg[v].z = w[2]; reg[v].w = w[3];
         }
      }
   }
   __device__ __forceinline__ void stash(uint16_t *buffer) const
   {
      if (KC)
      {
#pragma unroll
         for (int v = 0; v < NV; v++)
         {  uint32_t mn, k; where(v, mn, k);
            *reinterpret_cast<och_gu32x4 *>(buffer + (k / 8) * PLANE + mn * 8) = reg[v];
         }
      }
      else
      {  uint32_t mn, k; where(0, mn, k);
#pragma unroll
         for (int v = 0; v < NV; v++) *reinterpret_cast<och_gu32x4 *>(buffer + (k + v) * PITCH + mn) = reg[v];
      }
   }
   /* the same in single instructions, for loops that place every one of them by hand: load number v (whole tiles only),
      and store number `piece` of the NV = 8 that move the registers to LDS */
   /* address of load v = the slab's first element (the same for all threads: mat + element (mn0, k0)) + a step per v that is
      the same for all threads + the thread's own offset, which does not change from slab to slab: a scalar base and a
      32-bit vector offset, no 64-bit vector arithmetic in the loop */
   static __device__ __forceinline__ uint32_t thread_offset(int64_t ld)
   {  uint32_t mn, k; where(0, mn, k);
      return (uint32_t)((KC ? ((int64_t)k + (int64_t)mn * ld) : ((int64_t)mn + (int64_t)k * ld)) * 2);
   }
   static __device__ __forceinline__ const char *slab_base(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0)
   {  return mat + (KC ? ((int64_t)k0 + (int64_t)mn0 * ld) : ((int64_t)mn0 + (int64_t)k0 * ld)) * 2; }
   __device__ __forceinline__ void fetch_one(int v, const char *base, int64_t ld, uint32_t toff)
   {  /* where(v) - where(0): KC rows THREADS / (KT / 8) * v further on, !KC k further on by v */
      const int64_t step = KC ? (int64_t)(THREADS / (KT / 8)) * v * ld * 2 : (int64_t)v * ld * 2;
      reg[v] = *reinterpret_cast<const och_gu32x4 *>(base + step + toff);
   }
   static constexpr int PIECES = NV;                                    /* stores that move the registers to LDS */
   __device__ __forceinline__ void stash_one(uint16_t *buffer, int piece) const
   {  uint32_t mn, k; where(piece, mn, k);
      if (KC) *reinterpret_cast<och_gu32x4 *>(buffer + (k / 8) * PLANE + mn * 8) = reg[piece];
      else    *reinterpret_cast<och_gu32x4 *>(buffer + k * PITCH + mn) = reg[piece];
   }
   /* the eight k of slot `slot` that lane group `kg` (0 or 1) feeds to MFMA step `ks` (16 k per step) */
   static __device__ __forceinline__ och_h8 fragment(const uint16_t *buffer, int slot, int ks, int kg)
   {  och_h8 f;
      if (KC)
      {  const och_gu32x4 raw = *reinterpret_cast<const och_gu32x4 *>(buffer + (ks * 2 + kg) * PLANE + slot * 8);
         __builtin_memcpy(&f, &raw, 16);
      }
      else
      {  /* slot = first row of the tile + lane % 32; this lane reads rows (slot - lane % 16) + 4 (lane % 4) .. + 3 of
            k + (lane % 16) / 4 and receives row `slot` of k .. k + 3 */
         const int lane = threadIdx.x & 63;
         const uint16_t *at = buffer + (ks * 16 + kg * 8 + ((lane & 15) >> 2)) * PITCH + (slot - (lane & 15)) + 4 * (lane & 3);
         const och_i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) och_i16x4 *)at);
         const och_i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) och_i16x4 *)(at + 4 * PITCH));
         __builtin_memcpy(&f, &lo, 8);
         __builtin_memcpy(reinterpret_cast<char *>(&f) + 8, &hi, 8);
      }
      return f;
   }
};

/* PIPE: the main loop of the large tile with one wave per SIMD (four waves of 128 x 128): nothing hides a wave's memory
   and LDS latencies but the wave itself, so the loop is software-pipelined by hand. The fragments of MFMA step ks + 1 are
   read from LDS while the MFMAs of step ks run (two sets of fragment registers), the registers that hold slab s + 1 go
   to the other LDS buffer during steps 0 and 1 and the loads of slab s + 2 leave during step 2, and the one barrier of a
   slab stands in front of the last step's MFMAs, with the first fragment reads of the next slab right behind it. The
   loop body has no branches (slab numbers past the end are clamped to the last slab: its data is loaded and stored once
   more and never read), so the whole slab is one scheduling region. Only for tiles that lie inside the matrices. */
template <bool AKC, bool BKC, bool EDGE, int WM, int WN, int NWM, int NWN, int KT, bool PIPE = false>
__global__ __launch_bounds__(64 * NWM * NWN) void gemm_half_kernel(const HalfGemmParams p)
{
   constexpr int T = 32, THREADS = 64 * NWM * NWN;
   constexpr int BM = NWM * WM, BN = NWN * WN, TMS = WM / T, TNS = WN / T;
   typedef HalfSlab<AKC, EDGE, BM, KT, THREADS> LA;
   typedef HalfSlab<BKC, EDGE, BN, KT, THREADS> LB;
   constexpr int BUF = LA::SIZE + LB::SIZE;
   extern __shared__ __align__(16) uint16_t lds[];

   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const char *pA = p.A + oA, *pB = p.B + oB; char *pC = p.C + oC;
   /* (numbering the tiles so that every XCD owns a run of consecutive ones was measured and is slower: 8192^3 TN 958 -> 908 TFLOP/s) */
   const uint32_t tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   const int wm = (wave % NWM) * WM, wn = (wave / NWM) * WN;

   och_f32x16 acc[TMS][TNS];
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
#pragma unroll
         for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

   LA la; LB lb;
   uint32_t slab0 = 0, nslabs = (p.K + KT - 1) / KT;
   if (p.split_slabs)
   {  slab0 = blockIdx.z * p.split_slabs;
      nslabs = (slab0 + p.split_slabs < nslabs) ? p.split_slabs : (slab0 < nslabs ? nslabs - slab0 : 0);
   }
   if constexpr (PIPE)
   {  static_assert(!EDGE && KT == 64, "the pipelined loop is for whole tiles and slabs of 64");
      och_h8 fa[2][TMS], fb[2][TNS];
      const int arow = wm + lane % T, brow = wn + lane % T, kg = lane / T;
      const uint32_t toffA = LA::thread_offset(p.ldA), toffB = LB::thread_offset(p.ldB);
#define OCH_FRAGS(SET, AS, BS, KS)                                                                        \
      do { _Pragma("unroll") for (int i = 0; i < TMS; i++) fa[SET][i] = LA::fragment(AS, arow + i * T, KS, kg);      \
           _Pragma("unroll") for (int j = 0; j < TNS; j++) fb[SET][j] = LB::fragment(BS, brow + j * T, KS, kg); } while (0)
#define OCH_MFMAS(SET)                                                                                    \
      do { _Pragma("unroll") for (int i = 0; i < TMS; i++)                                                \
           _Pragma("unroll") for (int j = 0; j < TNS; j++)                                                \
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[SET][i], fb[SET][j], acc[i][j], 0, 0, 0); } while (0)
      /* a step = CH chunks of two MFMAs; chunk q also reads its share of the TMS + TNS fragments of the next step and runs
         FIRST and SECOND (a share of the step's stores to LDS and loads from memory); a scheduling fence closes the chunk */
      constexpr int CH = TMS * TNS / 2, NF = TMS + TNS;
      static_assert(TNS % 2 == 0, "a chunk is two MFMAs of one row of tiles");
#define OCH_SHARE(q, N, I) for (int I = (q) * (N) / CH; I < ((q) + 1) * (N) / CH; I++)
#define OCH_STEP(CUR, NXT, AS, BS, KS, FIRST, SECOND)                                                                  \
      do { _Pragma("unroll") for (int q = 0; q < CH; q++)                                                             \
           {  _Pragma("unroll") OCH_SHARE(q, NF, f)                                                                    \
              {  if (f < TMS) fa[NXT][f < TMS ? f : 0] = LA::fragment(AS, arow + f * T, KS, kg);                       \
                 else fb[NXT][f >= TMS ? f - TMS : 0] = LB::fragment(BS, brow + (f - TMS) * T, KS, kg);                \
              }                                                                                                        \
              FIRST; SECOND;                                                                                           \
              acc[(2 * q) / TNS][(2 * q) % TNS] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[CUR][(2 * q) / TNS], fb[CUR][(2 * q) % TNS], acc[(2 * q) / TNS][(2 * q) % TNS], 0, 0, 0); \
              acc[(2 * q) / TNS][(2 * q) % TNS + 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[CUR][(2 * q) / TNS], fb[CUR][(2 * q) % TNS + 1], acc[(2 * q) / TNS][(2 * q) % TNS + 1], 0, 0, 0); \
              __builtin_amdgcn_sched_barrier(0);                                                                       \
           } } while (0)
      if (nslabs > 0)
      {  const uint32_t last = slab0 + nslabs - 1;
         la.fetch(pA, p.ldA, m0, slab0 * KT, p.M, p.K, p.alignedA);
         lb.fetch(pB, p.ldB, n0, slab0 * KT, p.N, p.K, p.alignedB);
         la.stash(lds); lb.stash(lds + LA::SIZE);
         {  /* the loads of the second slab leave in the order in which the loop issues them (A then B, pair by pair): the
               compiler's count of loads that may still be in flight at a store of the loop is the worse of the two ways
               into the loop, and with the loads here in any order every store of the loop waited for nearly all of them */
            const uint32_t s1 = (slab0 + 1 < last) ? slab0 + 1 : last;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int v = 0; v < LA::NV; v++)
            {  la.fetch_one(v, LA::slab_base(pA, p.ldA, m0, s1 * KT), p.ldA, toffA);
               __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int v = 0; v < LB::NV; v++)
            {  lb.fetch_one(v, LB::slab_base(pB, p.ldB, n0, s1 * KT), p.ldB, toffB);
               __builtin_amdgcn_sched_barrier(0);
            }
         }
         __syncthreads();
         OCH_FRAGS(0, lds, lds + LA::SIZE, 0);
         for (uint32_t s = 0; s < nslabs; s++)
         {  const uint16_t *As = lds + (s & 1) * BUF, *Bs = As + LA::SIZE;
            uint16_t *An = lds + ((s + 1) & 1) * BUF, *Bn = An + LA::SIZE;
            const uint32_t s2 = (slab0 + s + 2 < last) ? slab0 + s + 2 : last;
            const char *nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);
            /* Every step is eight chunks of two MFMAs; a chunk also issues one fragment read for the next step and two of the
               step's other memory instructions, and a scheduling fence closes it, so the instructions leave in this order.
               Step 0: slab s + 1 of A goes from its registers to LDS (chunks 0-3) and slab s + 2 of A is asked for (chunks
               4-7), a slab ahead of its own store; step 1: the same for B; step 2: fragment reads only; then the barrier;
               step 3 reads the first fragments of the next slab. */
            OCH_STEP(0, 1, As, Bs, 1, _Pragma("unroll") OCH_SHARE(q, LA::PIECES, e) la.stash_one(An, e), (void)0);
            OCH_STEP(1, 0, As, Bs, 2, _Pragma("unroll") OCH_SHARE(q, LB::PIECES, e) lb.stash_one(Bn, e),
                                      _Pragma("unroll") OCH_SHARE(q, LA::NV, v) la.fetch_one(v, nextA, p.ldA, toffA));
            OCH_STEP(0, 1, As, Bs, 3, _Pragma("unroll") OCH_SHARE(q, LB::NV, v) lb.fetch_one(v, nextB, p.ldB, toffB), (void)0);
            __syncthreads();
            OCH_STEP(1, 0, An, Bn, 0, (void)0, (void)0);
         }
         __syncthreads();
      }
#undef OCH_FRAGS
#undef OCH_MFMAS
#undef OCH_STEP
#undef OCH_SHARE
   }
   else
   {
   /* registers hold the slab after the one in LDS: slab s + 1 is stored half way through the MFMAs of slab s (its stores
      run under the remaining MFMAs instead of in front of the barrier) and the loads of slab s + 2 are issued right after,
      a slab and a half before their data is needed */
   if (nslabs > 0)
   {  la.fetch(pA, p.ldA, m0, slab0 * KT, p.M, p.K, p.alignedA);
      lb.fetch(pB, p.ldB, n0, slab0 * KT, p.N, p.K, p.alignedB);
      la.stash(lds); lb.stash(lds + LA::SIZE);
      if (nslabs > 1)
      {  la.fetch(pA, p.ldA, m0, (slab0 + 1) * KT, p.M, p.K, p.alignedA);
         lb.fetch(pB, p.ldB, n0, (slab0 + 1) * KT, p.N, p.K, p.alignedB);
      }
   }
   __syncthreads();
   for (uint32_t s = 0; s < nslabs; s++)
   {  const uint16_t *As = lds + (s & 1) * BUF, *Bs = As + LA::SIZE;
#pragma unroll
      for (int ks = 0; ks < KT / 16; ks++)
      {  och_h8 a[TMS], b[TNS];
#pragma unroll
         for (int i = 0; i < TMS; i++) a[i] = LA::fragment(As, wm + i * T + lane % T, ks, lane / T);
#pragma unroll
         for (int j = 0; j < TNS; j++) b[j] = LB::fragment(Bs, wn + j * T + lane % T, ks, lane / T);
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int j = 0; j < TNS; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
         if (ks == KT / 32 - 1 && s + 1 < nslabs)
         {  uint16_t *An = lds + ((s + 1) & 1) * BUF;
            la.stash(An); lb.stash(An + LA::SIZE);
            if (s + 2 < nslabs)
            {  la.fetch(pA, p.ldA, m0, (slab0 + s + 2) * KT, p.M, p.K, p.alignedA);
               lb.fetch(pB, p.ldB, n0, (slab0 + s + 2) * KT, p.N, p.K, p.alignedB);
            }
         }
      }
      __syncthreads();
   }

   }
   const uint32_t row0 = LA::row_of_slot(wm + 4 * (lane >> 5)), col0 = LB::row_of_slot(wn + lane % T);
   if (p.split_slabs)
   {  /* raw sums of this K slice */
      float *plane = p.partial + (size_t)blockIdx.z * p.M * p.N;
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {  const uint32_t col = n0 + col0 + LB::row_step(j * T);
         if (col >= p.N) continue;
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {  const uint32_t row = m0 + row0 + LA::row_step(i * T + 8 * (r >> 2) + (r & 3));
               if (row < p.M) plane[(size_t)col * p.M + row] = acc[i][j][r];
            }
      }
      return;
   }

   /* epilogue: accumulator register r of lane l belongs to slot 8 * (r / 4) + 4 * (l / 32) + r % 4 of A and slot l % 32 of B
      within its 32 x 32 tile */
   half_t al = p.alpha, be = p.beta;
   if (p.alpha_dev) al = *reinterpret_cast<const half_t *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha);
   if (p.beta_dev)  be = *reinterpret_cast<const half_t *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);
   const float alpha = gemm_half_to_float(al), beta = gemm_half_to_float(be);
   /* this lane's part of tile (i, j): rows row0 + row_step(32 i + 8 (r / 4) + r % 4), column col0 + row_step(32 j); the
      slot offsets added here never carry out of a group of BM / 8 (BN / 8) slots, so the steps are compile-time numbers */
   if (beta == 0)
   {  /* C is only written: the rounded tile goes through LDS (the slab buffers are free after the last barrier), column
         by column with a pitch of BM + 8 halves, and leaves in 16-byte pieces that follow the columns of C */
      constexpr int CP = BM + 8;
      constexpr int PASSES = (BN * CP <= 2 * BUF) ? 1 : ((BN / 2) * CP <= 2 * BUF) ? 2 : 4;
      constexpr int CPASS = BN / PASSES;
      static_assert(CPASS * CP <= 2 * BUF, "the staged tile does not fit into the slab buffers");
      for (int h = 0; h < PASSES; h++)
      {  uint16_t *mine = lds + ((int)col0 - h * CPASS) * CP + row0;
#pragma unroll
         for (int j = 0; j < TNS; j++)
         {  if (PASSES > 1 && (col0 + LB::row_step(j * T)) / CPASS != (uint32_t)h) continue;
#pragma unroll
            for (int i = 0; i < TMS; i++)
#pragma unroll
               for (int r = 0; r < 16; r++)
                  mine[LB::row_step(j * T) * CP + LA::row_step(i * T + 8 * (r >> 2) + (r & 3))] = gemm_float_to_half(alpha * acc[i][j][r]).v;
         }
         __syncthreads();
         const uint32_t c0 = n0 + h * CPASS;
         const bool whole = !EDGE || (p.alignedC && (uint64_t)m0 + BM <= p.M && (uint64_t)c0 + CPASS <= p.N);
         for (uint32_t q = threadIdx.x; q < CPASS * (BM / 8); q += THREADS)
         {  const uint32_t c = q / (BM / 8), r8 = (q % (BM / 8)) * 8;
            const uint16_t *src = lds + c * CP + r8;
            char *dst = pC + ((int64_t)(m0 + r8) + (int64_t)(c0 + c) * p.ldC) * 2;
            if (whole) *reinterpret_cast<och_gu32x4 *>(dst) = *reinterpret_cast<const och_gu32x4 *>(src);
            else if (c0 + c < p.N)
            {
#pragma unroll
               for (int e = 0; e < 8; e++)
                  if (m0 + r8 + e < p.M) reinterpret_cast<uint16_t *>(dst)[e] = src[e];
            }
         }
         if (h + 1 < PASSES) __syncthreads();
      }
      return;
   }
   char *mine = pC + ((int64_t)(m0 + row0) + (int64_t)(n0 + col0) * p.ldC) * 2;
#pragma unroll
   for (int j = 0; j < TNS; j++)
   {  if (EDGE && n0 + col0 + LB::row_step(j * T) >= p.N) continue;
#pragma unroll
      for (int i = 0; i < TMS; i++)
#pragma unroll
         for (int r = 0; r < 16; r++)
         {
            const uint32_t dr = LA::row_step(i * T + 8 * (r >> 2) + (r & 3));
            if (EDGE && m0 + row0 + dr >= p.M) continue;
            half_t *c = reinterpret_cast<half_t *>(mine + ((int64_t)dr + (int64_t)LB::row_step(j * T) * p.ldC) * 2);
            *c = gemm_float_to_half(alpha * acc[i][j][r] + beta * gemm_half_to_float(*c));
         }
   }
}

/* adds the K slices of a split product in slice order, applies alpha / beta and rounds: one thread per element of C */
__global__ __launch_bounds__(256) void gemm_half_finish_kernel(const HalfGemmParams p, uint32_t slices)
{
   const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x, mn = (uint64_t)p.M * p.N;
   if (e >= mn) return;
   const uint32_t col = (uint32_t)(e / p.M), row = (uint32_t)(e - (uint64_t)col * p.M);
   float s = 0;
   uint32_t t = 0;
   for (; t + 7 < slices; t += 8)
   {  float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = p.partial[(size_t)(t + u) * mn + e];
#pragma unroll
      for (int u = 0; u < 8; u++) s += v[u];
   }
   for (; t < slices; t++) s += p.partial[(size_t)t * mn + e];
   const float alpha = gemm_half_to_float(p.alpha_dev ? *p.alpha_dev : p.alpha), beta = gemm_half_to_float(p.beta_dev ? *p.beta_dev : p.beta);
   half_t *c = reinterpret_cast<half_t *>(p.C) + ((int64_t)row + (int64_t)col * p.ldC);
   float v = alpha * s;
   if (beta != 0) v += beta * gemm_half_to_float(*c);
   *c = gemm_float_to_half(v);
}

template <int WM, int WN, int NWM, int NWN, int KT, bool PIPE = false>
static int launch_gemm_half(const GemmArgs &g)
{
   constexpr int BM = NWM * WM, BN = NWN * WN, THREADS = 64 * NWM * NWN;
   HalfGemmParams p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host) { memcpy(&p.alpha, g.alpha, 2); memcpy(&p.beta, g.beta, 2); }
   else { p.alpha_dev = (const half_t *)g.alpha; p.beta_dev = (const half_t *)g.beta; }
   p.batch = g.batch;
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   p.tiles_m = (uint32_t)((g.M + BM - 1) / BM); p.tiles_n = (uint32_t)((g.N + BN - 1) / BN);
   const uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   auto aligned = [&](const void *ptr, ptrdiff_t ld, const int64_t *bs)
   {  bool ok = ((uintptr_t)ptr % 16 == 0) && (((int64_t)ld * 2) % 16 == 0);
      for (int d = 0; d < g.batch.nb; d++) ok = ok && (bs[d] % 16 == 0);
      return ok;
   };
   p.alignedA = aligned(g.A, g.ldA, g.batch.sA) ? 1 : 0; p.alignedB = aligned(g.B, g.ldB, g.batch.sB) ? 1 : 0;
   p.alignedC = aligned(g.C, g.ldC, g.batch.sC) ? 1 : 0;
   /* the pipelined loop keeps a thread's offset within a slab in 32 bits: columns further apart than 64 MB take the guarded kernel */
   const bool far = PIPE && ((int64_t)g.ldA * 2 >= (1 << 26) || (int64_t)g.ldB * 2 >= (1 << 26));
   const bool edge = far || !(g.M % BM == 0 && g.N % BN == 0 && g.K % KT == 0 && p.alignedA && p.alignedB && p.alignedC);
   /* few tiles and a long K: slices of K in grid z, at least 8 slabs each, about 512 blocks in all, partial sums within the workspace */
   uint32_t slices = 1;
   {  const uint64_t nslabs = (g.K + KT - 1) / KT;
      if (g.batch.nb == 0 && blocks < (uint64_t)gemm_compute_units() && nslabs >= 32)
      {  uint64_t want = (512 + blocks - 1) / blocks;
         if (want > nslabs / 8) want = nslabs / 8;
         const uint64_t fit = OCH_GEMM_WORKSPACE / ((uint64_t)g.M * g.N * sizeof(float));
         if (want > fit) want = fit;
         if (want > 65535) want = 65535;
         if (want >= 2)
         {  char *ws;
            if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
            p.split_slabs = (uint32_t)((nslabs + want - 1) / want);
            slices = (uint32_t)((nslabs + p.split_slabs - 1) / p.split_slabs);
            p.partial = reinterpret_cast<float *>(ws);
            if (slices < 2) { slices = 1; p.split_slabs = 0; p.partial = nullptr; }
         }
      }
   }
   const dim3 grid((unsigned)blocks, 1, slices > 1 ? slices : g.nz), block(THREADS);
   /* both LDS buffers; above 64 KB the kernel has to be told */
#define OCH_HGEMM_LAUNCH(AK, BK, EDGE)                                                                                   \
   do { auto kernel = gemm_half_kernel<AK, BK, EDGE, WM, WN, NWM, NWN, KT, PIPE && !(EDGE)>;                             \
        const size_t lds = 2 * 2 * (size_t)(HalfSlab<AK, EDGE, BM, KT, THREADS>::SIZE + HalfSlab<BK, EDGE, BN, KT, THREADS>::SIZE); \
        if (lds > 65536) OCH_CHECK_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kernel, grid, block, lds, g.stream, p); } while (0)
#define OCH_HGEMM_PICK(AK, BK) do { if (edge) OCH_HGEMM_LAUNCH(AK, BK, true); else OCH_HGEMM_LAUNCH(AK, BK, false); } while (0)
   if (!akc && !bkc) OCH_HGEMM_PICK(false, false);
   else if (!akc)    OCH_HGEMM_PICK(false, true);
   else if (!bkc)    OCH_HGEMM_PICK(true, false);
   else              OCH_HGEMM_PICK(true, true);
#undef OCH_HGEMM_PICK
#undef OCH_HGEMM_LAUNCH
   if (slices > 1)
      hipLaunchKernelGGL(gemm_half_finish_kernel, dim3((unsigned)(((uint64_t)g.M * g.N + 255) / 256)), dim3(256), 0, g.stream, p, slices);
   OCH_CHECK_LAUNCH();
   return 0;
}

/* returns 1 when the product is left to the generic kernel (K < 16). Small results run on the 64 x 64 tile with the part
   outside the matrices read as zero -- the matrix cores are fast enough for that to beat a scalar kernel -- and products
   with few tiles and a long K are cut along K.
   Measured at 8192^3 (NN / NT / TN / TT, TFLOP/s): 256 x 256 tiles with eight waves 798 / 908 / 1021 / 1005; with
   128 x 128 tiles and four waves the same kernel stays 15 - 25 % below that. 4096^3 (256 tiles of 256 x 256):
   793 / 653 / 720 / 696. A 256 x 256 tile with four waves of 128 x 128 (a third less LDS traffic per MFMA) measures the
   same. With the loads from memory, the LDS stores, the fragment reads and the barriers taken out one by one the TN
   product (850 before the loads were moved a slab and a half ahead) rises to 1017, 1169, 1366 and, with the bare MFMA loop left, 1495 TFLOP/s: that, not the nominal
   2500, is what the matrix cores sustain here, and the kernel runs at about two thirds of it. */
int gemm_half(const GemmArgs &g)
{
   if (g.K < 16) return 1;                      /* C <- beta C, and updates of so low a rank that writing C is all there is */
   static const GemmTileChoice choice[3] = { { 256, 256, 1.0 }, { 128, 128, 0.8 }, { 64, 64, 0.55 } };
   switch (gemm_pick_tile(g, choice, 3))
   {  case 0:
         /* whole aligned tiles: four waves of 128 x 128 with the hand-pipelined loop; otherwise eight waves of 64 x 128 */
         if (g.M % 256 == 0 && g.N % 256 == 0 && g.K % 64 == 0) return launch_gemm_half<128, 128, 2, 2, 64, true>(g);
         if (g.K % 64 == 0 && g.M >= 256 && g.N >= 256 && gemm_operands_aligned(g, 2))
         {  /* whole tiles first, on the pipelined loop; then the strip of columns to their right and the strip of rows below them */
            const size_t Mi = g.M - g.M % 256, Ni = g.N - g.N % 256;
            GemmArgs part = g;
            part.M = Mi; part.N = Ni;
            if (launch_gemm_half<128, 128, 2, 2, 64, true>(part) != 0) return -1;
            if (g.N > Ni)
            {  part = g; part.N = g.N - Ni;
               part.B = (const char *)g.B + (int64_t)Ni * (g.transB == 'N' ? (int64_t)g.ldB : 1) * 2;
               part.C = (char *)g.C + (int64_t)Ni * g.ldC * 2;
               if (gemm_half(part) != 0) return -1;          /* K >= 64: never left to the generic kernel */
            }
            if (g.M > Mi)
            {  part = g; part.M = g.M - Mi; part.N = Ni;
               part.A = (const char *)g.A + (int64_t)Mi * (g.transA == 'N' ? 1 : (int64_t)g.ldA) * 2;
               part.C = (char *)g.C + (int64_t)Mi * 2;
               if (gemm_half(part) != 0) return -1;
            }
            return 0;
         }
         return launch_gemm_half<64, 128, 4, 2, 64>(g);
      case 1:
         /* whole 128 x 128 tiles take the pipelined loop too (2048^3: 400 -> 480 TFLOP/s, 3072^3: 500 -> 585) */
         if (g.M % 128 == 0 && g.N % 128 == 0 && g.K % 64 == 0) return launch_gemm_half<64, 64, 2, 2, 64, true>(g);
         return launch_gemm_half<64, 64, 2, 2, 64>(g);
      default: return launch_gemm_half<32, 32, 2, 2, 64>(g);
   }
}

} /* namespace och */
