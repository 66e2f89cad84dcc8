/* 8-bit integer and bool GEMM on the matrix cores: C <- alpha * op(A) * op(B) + beta * C, column-major.
 *
 * The reference multiplies integer matrices with its own tiled kernel (solid/src/core/gpu/template_blas.cu:99-160), in
 * wrap-around arithmetic of the element type; bool uses OR for + and AND for *. For int8 and uint8 only the low eight
 * bits of every sum matter, and those do not depend on whether the bytes are read as signed or unsigned, nor on the
 * sums wrapping at 32 bits: v_mfma_i32_32x32x32_i8 (signed 8-bit products, 32-bit sums) gives them exactly. For bool the
 * bytes are normalised to 0 / 1 when they are loaded, the sum counts the pairs that are both set, and the result is
 * "count non-zero".
 *
 * Structure as in the half-precision kernel: a block of NWM x NWN waves owns a tile of C, K steps of 128, slab s + 1 is
 * stored to the other LDS buffer half way through the MFMAs of slab s and the loads of slab s + 2 follow at once. LDS
 * holds an operand that is contiguous along k as 16-byte chunks of 16 k, chunk-major; one that is contiguous along m / n
 * as it lies in memory, and its fragments come out of transposing LDS reads (ds_read_b64_tr_b8).
 */
#include "och_gemm.h"

namespace och {

typedef int och_i32x4  __attribute__((ext_vector_type(4)));
typedef int och_i32x16 __attribute__((ext_vector_type(16)));
typedef int och_i32x2  __attribute__((ext_vector_type(2)));

struct ByteGemmParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements (bytes) */
   uint32_t M, N, K;
   uint8_t  alpha, beta;                /* when the scalars live in host memory */
   const uint8_t *alpha_dev, *beta_dev; /* non-null: read the scalar from device memory */
   int      alignedA, alignedB, alignedC;
   uint32_t tiles_m, tiles_n;
   GemmBatch batch;
   uint32_t split_slabs;                /* K slices in grid z, raw 32-bit sums in partial[z] (dense M x N planes) */
   int     *partial;
};

/* bytes that are not zero become 1 */
__device__ __forceinline__ uint32_t bool_bytes(uint32_t x)
{  return ((((x & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | x) & 0x80808080u) >> 7; }

/* Moves a BMN x KT slab of an operand (1-byte elements) from memory to registers and on to LDS, 16 bytes at a time, and
   reads MFMA fragments (sixteen consecutive k of one row per lane) from there.
   KC (contiguous along k in memory): a thread loads one chunk of 16 k of one row; LDS holds [chunk of 16 k][row][16 bytes],
   32 bytes of padding after every chunk plane; a fragment is one 16-byte read.
   !KC (contiguous along the row index): a thread loads 16 neighbouring rows of one k, for NV consecutive k, and LDS holds
   the slab as it lies in memory, [k][row] with a pitch of BMN + 16 bytes. The fragments come out of transposing reads
   (ds_read_b64_tr_b8): in every group of 16 lanes, lanes 2 e and 2 e + 1 read 16 neighbouring rows of k + e, and lane i of
   the group receives row i of k .. k + 7; two such reads make the sixteen k of a fragment. */
template <bool KC, bool EDGE, bool BOOL, int BMN, int KT, int THREADS>
struct ByteSlab
{
   static constexpr int NV = BMN * KT / 16 / THREADS;                  /* 16-byte loads per thread */
   static constexpr int G = BMN / 16;                                  /* groups of 16 rows */
   static constexpr int PLANE = BMN * 16 + 32;                         /* KC: bytes per chunk plane */
   static constexpr int PITCH = BMN + 16;                              /* !KC: bytes from one k to the next; 16 more than the rows so that the eight k of a transposing read meet different banks */
   static constexpr int SIZE = KC ? (KT / 16) * PLANE : KT * PITCH;    /* bytes per LDS buffer */
   static_assert(NV >= 1 && (BMN * KT) % (16 * THREADS) == 0, "slab does not divide among the threads");
   och_gu32x4 reg[NV];

   /* LDS slot -> row of the tile: the same for both layouts (kept as the one place that says so) */
   static __device__ __forceinline__ uint32_t row_of_slot(uint32_t slot) { return slot; }
   static constexpr uint32_t row_step(uint32_t o) { return o; }
   static __device__ __forceinline__ void where(int v, uint32_t &mn, uint32_t &k)
   {  if (!KC) { mn = (threadIdx.x % G) * 16; k = (threadIdx.x / G) * NV + v; }
      else     { const uint32_t q = threadIdx.x + THREADS * v; k = (q % (KT / 16)) * 16; mn = q / (KT / 16); }
   }
   /* element (mn, k) of op(.) lives at mn + k * ld (!KC) or k + mn * ld (KC) */
   __device__ __forceinline__ void fetch(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0, uint32_t MN, uint32_t K, int aligned)
   {
#pragma unroll
      for (int v = 0; v < NV; v++)
      {  uint32_t mn, k; where(v, mn, k);
         const int64_t gm = (int64_t)mn0 + mn, gk = (int64_t)k0 + k;
         const char *at = mat + (KC ? (gk + gm * ld) : (gm + gk * ld));
         bool whole = true;
         if (EDGE) whole = aligned && (KC ? (gm < (int64_t)MN && gk + 16 <= (int64_t)K) : (gk < (int64_t)K && gm + 16 <= (int64_t)MN));
         if (whole) reg[v] = *reinterpret_cast<const och_gu32x4 *>(at);
         else
         {  uint32_t w[4] = { 0, 0, 0, 0 };
            const bool some = KC ? (gm < (int64_t)MN && gk < (int64_t)K) : (gk < (int64_t)K && gm < (int64_t)MN);
            if (some)
            {
#pragma unroll
               for (int e = 0; e < 16; e++)
               {  const bool ok = KC ? (gk + e < (int64_t)K) : (gm + e < (int64_t)MN);
                  if (ok) w[e >> 2] |= (uint32_t)*reinterpret_cast<const uint8_t *>(at + e) << (8 * (e & 3));
               }
            }
            reg[v].x = w[0]; reg[v].y = w[1]; reg[v].z = w[2]; reg[v].w = w[3];
         }
         if (BOOL) { reg[v].x = bool_bytes(reg[v].x); reg[v].y = bool_bytes(reg[v].y); reg[v].z = bool_bytes(reg[v].z); reg[v].w = bool_bytes(reg[v].w); }
      }
   }
   __device__ __forceinline__ void stash(char *buffer) const
   {
      if (KC)
      {
#pragma unroll
         for (int v = 0; v < NV; v++)
         {  uint32_t mn, k; where(v, mn, k);
            *reinterpret_cast<och_gu32x4 *>(buffer + (k / 16) * PLANE + mn * 16) = reg[v];
         }
      }
      else
      {  uint32_t mn, k; where(0, mn, k);
#pragma unroll
         for (int v = 0; v < NV; v++) *reinterpret_cast<och_gu32x4 *>(buffer + (k + v) * PITCH + mn) = reg[v];
      }
   }
   /* The same in single instructions, for the loop that places every one of them by hand (whole tiles, no bool): load
      number v as a scalar base (the slab's first element, the same for all threads) + a step per v + the thread's own
      offset, which does not change from slab to slab; and store number `piece` of the PIECES that move the registers to LDS */
   static constexpr int PIECES = NV;
   static __device__ __forceinline__ uint32_t thread_offset(int64_t ld)
   {  uint32_t mn, k; where(0, mn, k);
      return (uint32_t)(KC ? ((int64_t)k + (int64_t)mn * ld) : ((int64_t)mn + (int64_t)k * ld));
   }
   static __device__ __forceinline__ const char *slab_base(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0)
   {  return mat + (KC ? ((int64_t)k0 + (int64_t)mn0 * ld) : ((int64_t)mn0 + (int64_t)k0 * ld)); }
   __device__ __forceinline__ void fetch_one(int v, const char *base, int64_t ld, uint32_t toff)
   {  const int64_t step = KC ? (int64_t)(THREADS / (KT / 16)) * v * ld : (int64_t)v * ld;
      reg[v] = *reinterpret_cast<const och_gu32x4 *>(base + step + toff);
   }
   __device__ __forceinline__ void stash_one(char *buffer, int piece) const
   {  uint32_t mn, k; where(piece, mn, k);
      if (KC) *reinterpret_cast<och_gu32x4 *>(buffer + (k / 16) * PLANE + mn * 16) = reg[piece];
      else    *reinterpret_cast<och_gu32x4 *>(buffer + k * PITCH + mn) = reg[piece];
   }
   /* the sixteen k of slot `slot` that lane group `kg` (0 or 1) feeds to MFMA step `ks` (32 k per step) */
   static __device__ __forceinline__ och_i32x4 fragment(const char *buffer, int slot, int ks, int kg)
   {  och_i32x4 f;
      if (KC)
      {  const och_gu32x4 raw = *reinterpret_cast<const och_gu32x4 *>(buffer + (ks * 2 + kg) * PLANE + slot * 16);
         __builtin_memcpy(&f, &raw, 16);
      }
      else
      {  /* slot = first row of the tile + lane % 32; this lane reads rows (slot - lane % 16) + 8 (lane % 2) .. + 7 of
            k + (lane % 16) / 2 and receives row `slot` of k .. k + 7 */
         const int lane = threadIdx.x & 63;
         const char *at = buffer + (ks * 32 + kg * 16 + ((lane & 15) >> 1)) * PITCH + (slot - (lane & 15)) + 8 * (lane & 1);
         const och_i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) och_i32x2 *)at);
         const och_i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) och_i32x2 *)(at + 8 * PITCH));
         f.x = lo.x; f.y = lo.y; f.z = hi.x; f.w = hi.y;
      }
      return f;
   }
};

/* alpha * s + beta * c in the arithmetic of the element type */
template <bool BOOL> __device__ __forceinline__ uint8_t byte_finish(int s, uint8_t alpha, uint8_t beta, uint8_t c, bool use_c)
{  if (BOOL) return (uint8_t)((((s != 0) && alpha) || (use_c && beta && c)) ? 1 : 0);
   return (uint8_t)((uint32_t)alpha * (uint32_t)s + (use_c ? (uint32_t)beta * (uint32_t)c : 0u));
}

/* PIPE: the hand-scheduled main loop of the half-precision kernel (gemm_half_kernel), for whole 256 x 256 tiles of int8 /
   uint8 with four waves of 128 x 128: fragments one MFMA step ahead in a second set of registers, the stores of slab s + 1
   to LDS and the loads of slab s + 2 spread one per chunk of two MFMAs over steps 0 to 2, one barrier per slab in front of
   the last step, no branches in the loop body (slab numbers past the end are clamped). */
template <bool AKC, bool BKC, bool EDGE, bool BOOL, int WM, int WN, int NWM, int NWN, int KT, bool PIPE = false>
__global__ __launch_bounds__(64 * NWM * NWN) void gemm_byte_kernel(const ByteGemmParams p)
{
   constexpr int T = 32, THREADS = 64 * NWM * NWN;
   constexpr int BM = NWM * WM, BN = NWN * WN, TMS = WM / T, TNS = WN / T;
   typedef ByteSlab<AKC, EDGE, BOOL, BM, KT, THREADS> LA;
   typedef ByteSlab<BKC, EDGE, BOOL, BN, KT, THREADS> LB;
   constexpr int BUF = LA::SIZE + LB::SIZE;
   extern __shared__ __align__(16) char lds_bytes[];
   char *lds = lds_bytes;

   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const char *pA = p.A + oA, *pB = p.B + oB; char *pC = p.C + oC;
   const uint32_t tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   const int wm = (wave % NWM) * WM, wn = (wave / NWM) * WN;

   och_i32x16 acc[TMS][TNS];
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
   {  static_assert(!EDGE && !BOOL && KT == 128, "the pipelined loop is for whole tiles of 8-bit integers and slabs of 128");
      och_i32x4 fa[2][TMS], fb[2][TNS];
      const int arow = wm + lane % T, brow = wn + lane % T, kg = lane / T;
      const uint32_t toffA = LA::thread_offset(p.ldA), toffB = LB::thread_offset(p.ldB);
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
              acc[(2 * q) / TNS][(2 * q) % TNS] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[CUR][(2 * q) / TNS], fb[CUR][(2 * q) % TNS], acc[(2 * q) / TNS][(2 * q) % TNS], 0, 0, 0); \
              acc[(2 * q) / TNS][(2 * q) % TNS + 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[CUR][(2 * q) / TNS], fb[CUR][(2 * q) % TNS + 1], acc[(2 * q) / TNS][(2 * q) % TNS + 1], 0, 0, 0); \
              __builtin_amdgcn_sched_barrier(0);                                                                       \
           } } while (0)
      if (nslabs > 0)
      {  const uint32_t last = slab0 + nslabs - 1;
         la.fetch(pA, p.ldA, m0, slab0 * KT, p.M, p.K, p.alignedA);
         lb.fetch(pB, p.ldB, n0, slab0 * KT, p.N, p.K, p.alignedB);
         la.stash(lds); lb.stash(lds + LA::SIZE);
         {  /* in the order of the loop, so that the compiler's count of loads in flight at the loop's stores is exact */
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
#pragma unroll
         for (int i = 0; i < TMS; i++) fa[0][i] = LA::fragment(lds, arow + i * T, 0, kg);
#pragma unroll
         for (int j = 0; j < TNS; j++) fb[0][j] = LB::fragment(lds + LA::SIZE, brow + j * T, 0, kg);
         for (uint32_t s = 0; s < nslabs; s++)
         {  const char *As = lds + (s & 1) * BUF, *Bs = As + LA::SIZE;
            char *An = lds + ((s + 1) & 1) * BUF, *Bn = An + LA::SIZE;
            const uint32_t s2 = (slab0 + s + 2 < last) ? slab0 + s + 2 : last;
            const char *nextA = LA::slab_base(pA, p.ldA, m0, s2 * KT), *nextB = LB::slab_base(pB, p.ldB, n0, s2 * KT);
            OCH_STEP(0, 1, As, Bs, 1, _Pragma("unroll") OCH_SHARE(q, LA::PIECES, e) la.stash_one(An, e), (void)0);
            OCH_STEP(1, 0, As, Bs, 2, _Pragma("unroll") OCH_SHARE(q, LB::PIECES, e) lb.stash_one(Bn, e),
                                      _Pragma("unroll") OCH_SHARE(q, LA::NV, v) la.fetch_one(v, nextA, p.ldA, toffA));
            OCH_STEP(0, 1, As, Bs, 3, _Pragma("unroll") OCH_SHARE(q, LB::NV, v) lb.fetch_one(v, nextB, p.ldB, toffB), (void)0);
            __syncthreads();
            OCH_STEP(1, 0, An, Bn, 0, (void)0, (void)0);
         }
         __syncthreads();
      }
#undef OCH_STEP
#undef OCH_SHARE
   }
   else
   {
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
   {  const char *As = lds + (s & 1) * BUF, *Bs = As + LA::SIZE;
#pragma unroll
      for (int ks = 0; ks < KT / 32; ks++)
      {  och_i32x4 a[TMS], b[TNS];
#pragma unroll
         for (int i = 0; i < TMS; i++) a[i] = LA::fragment(As, wm + i * T + lane % T, ks, lane / T);
#pragma unroll
         for (int j = 0; j < TNS; j++) b[j] = LB::fragment(Bs, wn + j * T + lane % T, ks, lane / T);
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int j = 0; j < TNS; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
         if (ks == KT / 64 - 1 && s + 1 < nslabs)
         {  char *An = lds + ((s + 1) & 1) * BUF;
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
   /* accumulator register r of lane l belongs to slot 8 * (r / 4) + 4 * (l / 32) + r % 4 of A and slot l % 32 of B within
      its 32 x 32 tile; the slot offsets added below never carry out of a group of BM / 16 (BN / 16) slots */
   const uint32_t row0 = LA::row_of_slot(wm + 4 * (lane >> 5)), col0 = LB::row_of_slot(wn + lane % T);
   if (p.split_slabs)
   {  int *plane = p.partial + (size_t)blockIdx.z * p.M * p.N;
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

   uint8_t alpha = p.alpha, beta = p.beta;
   if (p.alpha_dev) alpha = *(p.alpha_dev + oAlpha);
   if (p.beta_dev)  beta = *(p.beta_dev + oBeta);
   if (beta == 0)
   {  /* C is only written: the tile goes through LDS, column by column with a pitch of BM + 16 bytes, and leaves in
         16-byte pieces that follow the columns of C */
      constexpr int CP = BM + 16;
      static_assert(BN * CP <= 2 * BUF, "the staged tile does not fit into the slab buffers");
      char *mine = lds + col0 * CP + row0;
#pragma unroll
      for (int j = 0; j < TNS; j++)
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
               mine[LB::row_step(j * T) * CP + LA::row_step(i * T + 8 * (r >> 2) + (r & 3))] = (char)byte_finish<BOOL>(acc[i][j][r], alpha, 0, 0, false);
      __syncthreads();
      const bool whole = !EDGE || (p.alignedC && (uint64_t)m0 + BM <= p.M && (uint64_t)n0 + BN <= p.N);
      for (uint32_t q = threadIdx.x; q < BN * (BM / 16); q += THREADS)
      {  const uint32_t c = q / (BM / 16), r16 = (q % (BM / 16)) * 16;
         const char *src = lds + c * CP + r16;
         char *dst = pC + (int64_t)(m0 + r16) + (int64_t)(n0 + c) * p.ldC;
         if (whole) *reinterpret_cast<och_gu32x4 *>(dst) = *reinterpret_cast<const och_gu32x4 *>(src);
         else if (n0 + c < p.N)
         {
#pragma unroll
            for (int e = 0; e < 16; e++)
               if (m0 + r16 + e < p.M) dst[e] = src[e];
         }
      }
      return;
   }
   char *mine = pC + (int64_t)(m0 + row0) + (int64_t)(n0 + col0) * p.ldC;
#pragma unroll
   for (int j = 0; j < TNS; j++)
   {  if (EDGE && n0 + col0 + LB::row_step(j * T) >= p.N) continue;
#pragma unroll
      for (int i = 0; i < TMS; i++)
#pragma unroll
         for (int r = 0; r < 16; r++)
         {  const uint32_t dr = LA::row_step(i * T + 8 * (r >> 2) + (r & 3));
            if (EDGE && m0 + row0 + dr >= p.M) continue;
            uint8_t *c = reinterpret_cast<uint8_t *>(mine + (int64_t)dr + (int64_t)LB::row_step(j * T) * p.ldC);
            *c = byte_finish<BOOL>(acc[i][j][r], alpha, beta, *c, true);
         }
   }
}

/* adds the K slices of a split product in slice order and applies alpha / beta: one thread per element of C */
template <bool BOOL>
__global__ __launch_bounds__(256) void gemm_byte_finish_kernel(const ByteGemmParams p, uint32_t slices)
{
   const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x, mn = (uint64_t)p.M * p.N;
   if (e >= mn) return;
   const uint32_t col = (uint32_t)(e / p.M), row = (uint32_t)(e - (uint64_t)col * p.M);
   int s = 0;
   for (uint32_t t = 0; t < slices; t++)
   {  const int v = p.partial[(size_t)t * mn + e];
      s = BOOL ? (s | v) : (int)((uint32_t)s + (uint32_t)v);
   }
   const uint8_t alpha = p.alpha_dev ? *p.alpha_dev : p.alpha, beta = p.beta_dev ? *p.beta_dev : p.beta;
   uint8_t *c = reinterpret_cast<uint8_t *>(p.C) + ((int64_t)row + (int64_t)col * p.ldC);
   *c = byte_finish<BOOL>(s, alpha, beta, beta ? *c : (uint8_t)0, beta != 0);
}

template <bool BOOL, int WM, int WN, int NWM, int NWN, int KT, bool PIPE = false>
static int launch_gemm_byte(const GemmArgs &g)
{
   constexpr int BM = NWM * WM, BN = NWN * WN, THREADS = 64 * NWM * NWN;
   ByteGemmParams p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host) { memcpy(&p.alpha, g.alpha, 1); memcpy(&p.beta, g.beta, 1); }
   else { p.alpha_dev = (const uint8_t *)g.alpha; p.beta_dev = (const uint8_t *)g.beta; }
   p.batch = g.batch;
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   p.tiles_m = (uint32_t)((g.M + BM - 1) / BM); p.tiles_n = (uint32_t)((g.N + BN - 1) / BN);
   const uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   auto aligned = [&](const void *ptr, ptrdiff_t ld, const int64_t *bs)
   {  bool ok = ((uintptr_t)ptr % 16 == 0) && ((int64_t)ld % 16 == 0);
      for (int d = 0; d < g.batch.nb; d++) ok = ok && (bs[d] % 16 == 0);
      return ok;
   };
   p.alignedA = aligned(g.A, g.ldA, g.batch.sA) ? 1 : 0; p.alignedB = aligned(g.B, g.ldB, g.batch.sB) ? 1 : 0;
   p.alignedC = aligned(g.C, g.ldC, g.batch.sC) ? 1 : 0;
   /* the pipelined loop keeps a thread's offset within a slab in 32 bits: columns further apart than 64 MB take the guarded kernel */
   const bool far = PIPE && ((int64_t)g.ldA * 1 >= (1 << 26) || (int64_t)g.ldB * 1 >= (1 << 26));
   const bool edge = far || !(g.M % BM == 0 && g.N % BN == 0 && g.K % KT == 0 && p.alignedA && p.alignedB && p.alignedC);
   /* few tiles and a long K: slices of K in grid z, at least 8 slabs each, about 512 blocks in all, partial sums within the workspace */
   uint32_t slices = 1;
   {  const uint64_t nslabs = (g.K + KT - 1) / KT;
      if (g.batch.nb == 0 && blocks < (uint64_t)gemm_compute_units() && nslabs >= 32)
      {  uint64_t want = (512 + blocks - 1) / blocks;
         if (want > nslabs / 8) want = nslabs / 8;
         const uint64_t fit = OCH_GEMM_WORKSPACE / ((uint64_t)g.M * g.N * sizeof(int));
         if (want > fit) want = fit;
         if (want > 65535) want = 65535;
         if (want >= 2)
         {  char *ws;
            if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
            p.split_slabs = (uint32_t)((nslabs + want - 1) / want);
            slices = (uint32_t)((nslabs + p.split_slabs - 1) / p.split_slabs);
            p.partial = reinterpret_cast<int *>(ws);
            if (slices < 2) { slices = 1; p.split_slabs = 0; p.partial = nullptr; }
         }
      }
   }
   const dim3 grid((unsigned)blocks, 1, slices > 1 ? slices : g.nz), block(THREADS);
#define OCH_BGEMM_LAUNCH(AK, BK, EDGE)                                                                                    \
   do { auto kernel = gemm_byte_kernel<AK, BK, EDGE, BOOL, WM, WN, NWM, NWN, KT, PIPE && !(EDGE) && !BOOL>;               \
        const size_t lds = 2 * (size_t)(ByteSlab<AK, EDGE, BOOL, BM, KT, THREADS>::SIZE + ByteSlab<BK, EDGE, BOOL, BN, KT, THREADS>::SIZE); \
        if (lds > 65536) OCH_CHECK_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL(kernel, grid, block, lds, g.stream, p); } while (0)
#define OCH_BGEMM_PICK(AK, BK) do { if (edge) OCH_BGEMM_LAUNCH(AK, BK, true); else OCH_BGEMM_LAUNCH(AK, BK, false); } while (0)
   if (!akc && !bkc) OCH_BGEMM_PICK(false, false);
   else if (!akc)    OCH_BGEMM_PICK(false, true);
   else if (!bkc)    OCH_BGEMM_PICK(true, false);
   else              OCH_BGEMM_PICK(true, true);
#undef OCH_BGEMM_PICK
#undef OCH_BGEMM_LAUNCH
   if (slices > 1)
      hipLaunchKernelGGL(gemm_byte_finish_kernel<BOOL>, dim3((unsigned)(((uint64_t)g.M * g.N + 255) / 256)), dim3(256), 0, g.stream, p, slices);
   OCH_CHECK_LAUNCH();
   return 0;
}

/* returns 1 when the product is left to the generic kernel (K < 32) */
template <bool BOOL> static int gemm_byte_pick(const GemmArgs &g)
{
   if (g.K < 32) return 1;
   static const GemmTileChoice choice[3] = { { 256, 256, 1.0 }, { 128, 128, 0.8 }, { 64, 64, 0.55 } };
   switch (gemm_pick_tile(g, choice, 3))
   {  case 0:
         /* whole tiles of 8-bit integers: four waves of 128 x 128 with the hand-pipelined loop; otherwise eight waves of 64 x 128 */
         if (!BOOL && g.M % 256 == 0 && g.N % 256 == 0 && g.K % 128 == 0) return launch_gemm_byte<BOOL, 128, 128, 2, 2, 128, true>(g);
         if (!BOOL && g.K % 128 == 0 && g.M >= 256 && g.N >= 256 && gemm_operands_aligned(g, 1))
         {  /* whole tiles first, on the pipelined loop; then the strip of columns to their right and the strip of rows below them */
            const size_t Mi = g.M - g.M % 256, Ni = g.N - g.N % 256;
            GemmArgs part = g;
            part.M = Mi; part.N = Ni;
            if (launch_gemm_byte<BOOL, 128, 128, 2, 2, 128, true>(part) != 0) return -1;
            if (g.N > Ni)
            {  part = g; part.N = g.N - Ni;
               part.B = (const char *)g.B + (int64_t)Ni * (g.transB == 'N' ? (int64_t)g.ldB : 1);
               part.C = (char *)g.C + (int64_t)Ni * g.ldC;
               if (gemm_byte_pick<BOOL>(part) != 0) return -1;        /* K >= 128: never left to the generic kernel */
            }
            if (g.M > Mi)
            {  part = g; part.M = g.M - Mi; part.N = Ni;
               part.A = (const char *)g.A + (int64_t)Mi * (g.transA == 'N' ? 1 : (int64_t)g.ldA);
               part.C = (char *)g.C + (int64_t)Mi;
               if (gemm_byte_pick<BOOL>(part) != 0) return -1;
            }
            return 0;
         }
         return launch_gemm_byte<BOOL, 64, 128, 4, 2, 128>(g);
      case 1:
         if (!BOOL && g.M % 128 == 0 && g.N % 128 == 0 && g.K % 128 == 0) return launch_gemm_byte<BOOL, 64, 64, 2, 2, 128, true>(g);
         return launch_gemm_byte<BOOL, 64, 64, 2, 2, 128>(g);
      default: return launch_gemm_byte<BOOL, 32, 32, 2, 2, 128>(g);
   }
}
int gemm_int8(const GemmArgs &g) { return gemm_byte_pick<false>(g); }
int gemm_bool(const GemmArgs &g) { return gemm_byte_pick<true>(g); }

} /* namespace och */
