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
 * (column) per lane, so both operands are kept [row][k] in LDS (row pitch KT + 8 halves: the 16-byte reads of 16
 * neighbouring rows fall into distinct banks) and a fragment is one 16-byte LDS read. An operand that is contiguous
 * along k in memory ('T' for A, 'N' for B) arrives in that shape; one that is contiguous along m / n is transposed in
 * registers on its way to LDS. Which k a lane holds does not matter as long as A and B agree, and they do by construction.
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

/* Moves a BMN x KT slab of an operand (2-byte elements) from memory to registers and on to LDS, where it is kept
   [row][k] with a row pitch of KT + 8 halves; the 16-byte chunk c of row r sits at chunk position c ^ ((r / 16) mod 8).
   KC (contiguous along k in memory): a thread loads 16 bytes = 8 k of one row and stores them as they are.
   !KC (contiguous along the row index): a thread loads NV consecutive k for 8 neighbouring rows (16 bytes each),
   transposes the 8 x NV block in registers and stores NV k for each of the 8 rows. Neighbouring lanes hold rows that are
   8 apart; the chunk permutation spreads them over the banks (without it 16 lanes share a bank), and it leaves the
   fragment reads of 16 neighbouring rows, which the row pitch already keeps apart, as they are. */
template <bool KC, bool EDGE, int BMN, int KT, int THREADS>
struct HalfSlab
{
   static constexpr int NV = BMN * KT / 8 / THREADS;                   /* 16-byte loads per thread */
   static constexpr int PITCH = KT + 8;                                /* LDS row pitch in halves */
   static constexpr int SIZE = BMN * PITCH;                            /* halves per LDS buffer */
   static_assert(NV >= 1 && (BMN * KT) % (8 * THREADS) == 0, "slab does not divide among the threads");
   static_assert(KC || NV == 2 || NV == 4 || NV == 8, "the transposing loader needs 2, 4 or 8 k per thread");
   static_assert(KT == 64, "the chunk permutation assumes 8 chunks per row");
   static __device__ __forceinline__ uint32_t chunk_at(uint32_t row, uint32_t chunk) { return chunk ^ ((row >> 4) & 7); }
   och_gu32x4 reg[NV];

   static __device__ __forceinline__ void where(int v, uint32_t &mn, uint32_t &k)
   {  if (!KC) { mn = (threadIdx.x % (BMN / 8)) * 8; k = (threadIdx.x / (BMN / 8)) * NV + v; }
      else     { const uint32_t q = threadIdx.x + THREADS * v; k = (q % (KT / 8)) * 8; mn = q / (KT / 8); }
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
      if (KC)
      {
#pragma unroll
         for (int v = 0; v < NV; v++)
         {  uint32_t mn, k; where(v, mn, k);
            *reinterpret_cast<och_gu32x4 *>(plane + mn * PITCH + chunk_at(mn, k / 8) * 8) = reg[v];
         }
      }
      else
      {  constexpr int WD = NV / 2;                     /* 32-bit words per row: k pairs */
         uint32_t mn, k; where(0, mn, k);
         uint16_t *dst = plane + mn * PITCH + chunk_at(mn, k / 8) * 8 + k % 8;      /* mn is a multiple of 8: one chunk position for the 8 rows */
#pragma unroll
         for (int i = 0; i < 8; i++)
         {  uint32_t out[WD];
#pragma unroll
            for (int w = 0; w < WD; w++)
            {  const uint32_t x = reg[2 * w][i >> 1], y = reg[2 * w + 1][i >> 1];
               out[w] = (i & 1) ? ((x >> 16) | (y & 0xFFFF0000u)) : ((x & 0xFFFFu) | (y << 16));
            }
            if (WD == 1) *reinterpret_cast<uint32_t *>(dst + i * PITCH) = out[0];
            else if (WD == 2) { uint2 t; t.x = out[0]; t.y = out[WD > 1 ? 1 : 0]; *reinterpret_cast<uint2 *>(dst + i * PITCH) = t; }
            else { och_gu32x4 t; t.x = out[0]; t.y = out[WD > 1 ? 1 : 0]; t.z = out[WD > 2 ? 2 : 0]; t.w = out[WD > 3 ? 3 : 0]; *reinterpret_cast<och_gu32x4 *>(dst + i * PITCH) = t; }
         }
      }
   }
   /* the eight k of row `row` that lane group `kg` (0 or 1) feeds to MFMA step `ks` (16 k per step) */
   static __device__ __forceinline__ och_h8 fragment(const uint16_t *plane, int row, int ks, int kg)
   {  och_h8 f;
      const och_gu32x4 raw = *reinterpret_cast<const och_gu32x4 *>(plane + row * PITCH + chunk_at(row, ks * 2 + kg) * 8);
      __builtin_memcpy(&f, &raw, 16);
      return f;
   }
};

template <bool AKC, bool BKC, bool EDGE, int WM, int WN, int NWM, int NWN, int KT>
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

template <int WM, int WN, int NWM, int NWN, int KT>
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
   const bool edge = !(g.M % BM == 0 && g.N % BN == 0 && g.K % KT == 0 && p.alignedA && p.alignedB);
   const dim3 grid((unsigned)blocks, 1, g.nz), block(THREADS);
   /* both LDS buffers; above 64 KB the kernel has to be told */
#define OCH_HGEMM_LAUNCH(AK, BK, EDGE)                                                                                   \
   do { auto kernel = gemm_half_kernel<AK, BK, EDGE, WM, WN, NWM, NWN, KT>;                                              \
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
   OCH_CHECK_LAUNCH();
   return 0;
}

/* returns 1 when the product is left to the generic kernel (very small results or K).
   Measured at 8192^3 (NN / NT / TN / TT, TFLOP/s): 256 x 256 tiles with eight waves 711 / 758 / 904 / 846,
   128 x 128 tiles with four waves 610 / 608 / 791 / 737; at 4096^3 (256 tiles of 256 x 256) 661 / 556 / 650 / 621
   against 617 / 473 / 594 / 585. */
int gemm_half(const GemmArgs &g)
{
   if (g.M < 32 || g.N < 32 || g.K < 16) return 1;
   const uint64_t big = ((g.M + 255) / 256) * ((g.N + 255) / 256) * (uint64_t)g.nz;
   if (big >= 192) return launch_gemm_half<64, 128, 4, 2, 64>(g);
   if (!gemm_few_tiles(g, 128, 128)) return launch_gemm_half<64, 64, 2, 2, 64>(g);
   return launch_gemm_half<32, 32, 2, 2, 64>(g);
}

} /* namespace och */
