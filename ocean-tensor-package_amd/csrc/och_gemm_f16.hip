/* Half-precision GEMM on the matrix cores: C <- alpha * op(A) * op(B) + beta * C, column-major, half in memory.
 *
 * The reference multiplies half matrices with cublasHgemm where the device has it and otherwise converts the operands to
 * float, runs the float product and converts back (src/core/interface/tensor_itf.c:6388-6400,
 * src/core/gpu/op/tensor_blas_gpu.c:259-286). Here products of halves are accumulated in float by
 * v_mfma_f32_32x32x16_f16, alpha and beta are applied in float, and the result is rounded to half once with the
 * conversion every other operation uses -- the arithmetic of the float route.
 *
 * A block of four waves owns a (2*WM) x (2*WN) tile of C, each wave WM x WN of it as 32 x 32 MFMA tiles. Per K step of
 * KT = 32 the block stages slabs of op(A) and op(B) through LDS, loading slab s+1 from memory into registers before the
 * MFMAs of slab s and writing it to the other LDS buffer afterwards. An MFMA operand is eight consecutive k of one row
 * (column) per lane:
 *   - an operand that is contiguous along k in memory ('T' for A, 'N' for B) is kept [row][k] in LDS (row pitch KT + 8
 *     halves, so that the 16-byte reads of 16 neighbouring rows fall into distinct banks) and read with one 16-byte load;
 *   - an operand that is contiguous along m / n is kept [k][row] as it arrives and gathered with eight 2-byte loads.
 * Which k a lane holds does not matter as long as A and B agree, and they do by construction.
 */
#include "och_gemm.h"

namespace och {

typedef _Float16 och_h8 __attribute__((ext_vector_type(8)));

struct HalfGemmParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   half_t   alpha, beta;                /* when the scalars live in host memory */
   const half_t *alpha_dev, *beta_dev;  /* non-null: read the scalar from device memory */
   int      alignedA, alignedB;         /* base pointer, leading dimension and batch strides allow 128-bit loads */
   uint32_t tiles_m, tiles_n;
   GemmBatch batch;
};

#define OCH_HGEMM_KT 32

/* Moves a BMN x KT slab of an operand (2-byte elements) from memory to registers and on to LDS */
template <bool KC, bool EDGE, int BMN>
struct HalfSlab
{
   static constexpr int KT = OCH_HGEMM_KT;
   static constexpr int NV = BMN * KT / 8 / OCH_GEMM_THREADS;           /* 16-byte loads per thread */
   static constexpr int PITCH = (KC ? KT : BMN) + 8;                   /* LDS row pitch in halves */
   static constexpr int SIZE = (KC ? BMN : KT) * PITCH;                /* halves per LDS buffer */
   static_assert(NV >= 1 && (BMN * KT) % (8 * OCH_GEMM_THREADS) == 0, "slab does not divide among the threads");
   och_gu32x4 reg[NV];

   static __device__ __forceinline__ void where(int v, uint32_t &mn, uint32_t &k)
   {  const uint32_t q = threadIdx.x + OCH_GEMM_THREADS * v;
      if (!KC) { mn = (q % (BMN / 8)) * 8; k = q / (BMN / 8); }
      else     { k = (q % (KT / 8)) * 8;   mn = q / (KT / 8); }
   }
   /* element (mn, k) of op(.) lives at mn + k * ld (!KC) or k + mn * ld (KC) */
   __device__ __forceinline__ void fetch(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0, uint32_t MN, uint32_t K, int aligned)
   {
      const bool wide = !EDGE || (aligned && (uint64_t)mn0 + BMN <= MN && (uint64_t)k0 + KT <= K);
#pragma unroll
      for (int v = 0; v < NV; v++)
      {  uint32_t mn, k; where(v, mn, k);
         const int64_t gm = (int64_t)mn0 + mn, gk = (int64_t)k0 + k;
         if (wide) reg[v] = *reinterpret_cast<const och_gu32x4 *>(mat + (KC ? (gk + gm * ld) : (gm + gk * ld)) * 2);
         else
         {  uint32_t w[4] = { 0, 0, 0, 0 };
#pragma unroll
            for (int e = 0; e < 8; e++)
            {  const int64_t em = gm + (KC ? 0 : e), ek = gk + (KC ? e : 0);
               if (em < (int64_t)MN && ek < (int64_t)K)
                  w[e >> 1] |= (uint32_t)*reinterpret_cast<const uint16_t *>(mat + (KC ? (ek + em * ld) : (em + ek * ld)) * 2) << (16 * (e & 1));
            }
            reg[v].x = w[0]; reg[v].y = w[1]; reg[v].z = w[2]; reg[v].w = w[3];
         }
      }
   }
   __device__ __forceinline__ void stash(uint16_t *plane) const
   {
#pragma unroll
      for (int v = 0; v < NV; v++)
      {  uint32_t mn, k; where(v, mn, k);
         *reinterpret_cast<och_gu32x4 *>(plane + (KC ? (mn * PITCH + k) : (k * PITCH + mn))) = reg[v];
      }
   }
   /* the eight k of row `row` that lane group `kg` (0 or 1) feeds to MFMA step `ks` (16 k per step) */
   static __device__ __forceinline__ och_h8 fragment(const uint16_t *plane, int row, int ks, int kg)
   {  const int k = ks * 16 + kg * 8;
      och_h8 f;
      if (KC) { och_gu32x4 raw = *reinterpret_cast<const och_gu32x4 *>(plane + row * PITCH + k); __builtin_memcpy(&f, &raw, 16); }
      else
      {  uint16_t h[8];
#pragma unroll
         for (int e = 0; e < 8; e++) h[e] = plane[(k + e) * PITCH + row];
         __builtin_memcpy(&f, h, 16);
      }
      return f;
   }
};

template <bool AKC, bool BKC, bool EDGE, int WM, int WN>
__global__ __launch_bounds__(OCH_GEMM_THREADS, 2) void gemm_half_kernel(const HalfGemmParams p)
{
   constexpr int KT = OCH_HGEMM_KT, T = 32;
   constexpr int BM = 2 * WM, BN = 2 * WN, TMS = WM / T, TNS = WN / T;
   typedef HalfSlab<AKC, EDGE, BM> LA;
   typedef HalfSlab<BKC, EDGE, BN> LB;
   constexpr int BUF = LA::SIZE + LB::SIZE;
   __shared__ __align__(16) uint16_t lds[2 * BUF];

   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const char *pA = p.A + oA, *pB = p.B + oB; char *pC = p.C + oC;
   const uint32_t tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   const int wm = (wave & 1) * WM, wn = (wave >> 1) * WN;

   och_f32x16 acc[TMS][TNS];
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
#pragma unroll
         for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

   LA la; LB lb;
   const uint32_t nslabs = (p.K + KT - 1) / KT;
   if (nslabs > 0)
   {  la.fetch(pA, p.ldA, m0, 0, p.M, p.K, p.alignedA);
      lb.fetch(pB, p.ldB, n0, 0, p.N, p.K, p.alignedB);
      la.stash(lds); lb.stash(lds + LA::SIZE);
   }
   __syncthreads();
   for (uint32_t s = 0; s < nslabs; s++)
   {  const uint16_t *As = lds + (s & 1) * BUF, *Bs = As + LA::SIZE;
      const bool more = s + 1 < nslabs;
      if (more)
      {  la.fetch(pA, p.ldA, m0, (s + 1) * KT, p.M, p.K, p.alignedA);
         lb.fetch(pB, p.ldB, n0, (s + 1) * KT, p.N, p.K, p.alignedB);
      }
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
      }
      if (more)
      {  uint16_t *An = lds + ((s + 1) & 1) * BUF;
         la.stash(An); lb.stash(An + LA::SIZE);
      }
      __syncthreads();
   }

   /* epilogue: accumulator register r of lane l is C(8 * (r / 4) + 4 * (l / 32) + r % 4, l % 32) of its 32 x 32 tile */
   half_t al = p.alpha, be = p.beta;
   if (p.alpha_dev) al = *reinterpret_cast<const half_t *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha);
   if (p.beta_dev)  be = *reinterpret_cast<const half_t *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);
   const float alpha = half_to_float(al), beta = half_to_float(be);
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {  const uint32_t col = n0 + wn + j * T + lane % T;
#pragma unroll
         for (int r = 0; r < 16; r++)
         {  const uint32_t row = m0 + wm + i * T + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (EDGE && (row >= p.M || col >= p.N)) continue;
            half_t *c = reinterpret_cast<half_t *>(pC + ((int64_t)row + (int64_t)col * p.ldC) * 2);
            float v = alpha * acc[i][j][r];
            if (beta != 0) v += beta * half_to_float(*c);
            *c = float_to_half(v);
         }
      }
}

template <int WM, int WN>
static int launch_gemm_half(const GemmArgs &g)
{
   constexpr int BM = 2 * WM, BN = 2 * WN;
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
   const bool edge = !(g.M % BM == 0 && g.N % BN == 0 && g.K % OCH_HGEMM_KT == 0 && p.alignedA && p.alignedB);
   const dim3 grid((unsigned)blocks, 1, g.nz), block(OCH_GEMM_THREADS);
#define OCH_HGEMM_LAUNCH(AK, BK)                                                                               \
   do { if (edge) hipLaunchKernelGGL((gemm_half_kernel<AK, BK, true, WM, WN>), grid, block, 0, g.stream, p);   \
        else      hipLaunchKernelGGL((gemm_half_kernel<AK, BK, false, WM, WN>), grid, block, 0, g.stream, p); } while (0)
   if (!akc && !bkc) OCH_HGEMM_LAUNCH(false, false);
   else if (!akc)    OCH_HGEMM_LAUNCH(false, true);
   else if (!bkc)    OCH_HGEMM_LAUNCH(true, false);
   else              OCH_HGEMM_LAUNCH(true, true);
#undef OCH_HGEMM_LAUNCH
   OCH_CHECK_LAUNCH();
   return 0;
}

/* returns 1 when the product is left to the generic kernel (very small results or K) */
int gemm_half(const GemmArgs &g)
{
   if (g.M < 32 || g.N < 32 || g.K < 16) return 1;
   if (gemm_few_tiles(g, 128, 128)) return launch_gemm_half<32, 32>(g);
   return launch_gemm_half<64, 64>(g);
}

} /* namespace och */
