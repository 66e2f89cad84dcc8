/* GEMM kernels for gfx950: C <- alpha * op(A) * op(B) + beta * C, column-major.
 *
 * Replaces the cuBLAS dispatch of src/core/gpu/op/tensor_blas_gpu.c:132-231 (float, double,
 * cfloat, cdouble: MFMA kernels below) and the tiled integer kernels of
 * solid/src/core/gpu/template_blas.cu:99-160 (bool, integers, half: the generic kernel).
 *
 * MFMA kernel: a block of four waves owns a (2*WM) x (2*WN) tile of C; each wave a WM x WN
 * sub-tile made of v_mfma_f64_16x16x4_f64 / v_mfma_f32_32x32x2_f32 tiles held in registers.
 * Per K step the block stages a (2*WM) x KT slab of op(A) and a KT x (2*WN) slab of op(B)
 * through LDS in k-major order (As[k][m], Bs[k][n]); so both the "m/n-contiguous" and the
 * "k-contiguous" (transposed) memory layouts end up in the same LDS layout and the inner loop
 * does not depend on the transposition flags. Global loads of slab s+1 are issued before the
 * MFMAs of slab s and written to the other LDS buffer afterwards (one barrier per slab).
 * Complex types keep real and imaginary planes apart in LDS and use four real MFMAs per tile
 * (the sign of imag(A) is flipped in a register for the real part; conjugation flips the
 * sign when the plane is written).
 */
#pragma once
#include "och_common.h"
#include "och_dtypes.h"
#include "och_gemv.h"
#include <string.h>

namespace och {

typedef double och_f64x4  __attribute__((ext_vector_type(4)));
typedef float  och_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int och_gu32x4 __attribute__((ext_vector_type(4)));

/* One MFMA tile. Operands: lane l supplies A(row l % T, k = l / T) and B(k = l / T, col l % T);
   accumulator register r of lane l is C(acc_row(l, r), l % T). */
template <class R> struct Mfma;
template <> struct Mfma<double>
{  static constexpr int T = 16, TK = 4, NACC = 4;
   typedef och_f64x4 Acc;
   static __device__ __forceinline__ Acc mma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
   static __device__ __forceinline__ int acc_row(int lane, int r) { return 4 * r + (lane >> 4); }
};
template <> struct Mfma<float>
{  static constexpr int T = 32, TK = 2, NACC = 16;
   typedef och_f32x16 Acc;
   static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
   static __device__ __forceinline__ int acc_row(int lane, int r) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }
};

/* Batch of products in one launch (grid z): entry z is split into indices over `size`, and every operand --
   the scalars included when they live in device memory -- moves by its own byte stride per index (0: shared). */
#define OCH_GEMM_BATCH_DIMS 6
struct GemmBatch
{
   int      nb;                                   /* 0: a single product */
   uint32_t z0;                                   /* batch entry of grid z = 0 */
   uint32_t size[OCH_GEMM_BATCH_DIMS];
   int64_t  sA[OCH_GEMM_BATCH_DIMS], sB[OCH_GEMM_BATCH_DIMS], sC[OCH_GEMM_BATCH_DIMS];
   int64_t  sAlpha[OCH_GEMM_BATCH_DIMS], sBeta[OCH_GEMM_BATCH_DIMS];
};
__device__ __forceinline__ void gemm_batch_offsets(const GemmBatch &b, int64_t &oA, int64_t &oB, int64_t &oC, int64_t &oAlpha, int64_t &oBeta)
{  oA = oB = oC = oAlpha = oBeta = 0;
   if (b.nb == 0) return;
   uint32_t z = b.z0 + blockIdx.z;
   for (int d = 0; d < b.nb; d++)
   {  const uint32_t q = z / b.size[d], i = z - q * b.size[d]; z = q;
      oA += (int64_t)i * b.sA[d]; oB += (int64_t)i * b.sB[d]; oC += (int64_t)i * b.sC[d];
      oAlpha += (int64_t)i * b.sAlpha[d]; oBeta += (int64_t)i * b.sBeta[d];
   }
}

template <class R> struct GemmParams
{
   const char *A, *B; char *C;
   int64_t  ldA, ldB, ldC;              /* in elements */
   uint32_t M, N, K;
   R        alpha[2], beta[2];          /* (re, im) when the scalars live in host memory */
   const R *alpha_dev, *beta_dev;       /* non-null: read the scalar from device memory */
   int      conjA, conjB;
   int      alignedA, alignedB;        /* base pointer and leading dimension allow 128-bit loads */
   uint32_t tiles_m, tiles_n;
   GemmBatch batch;
   /* split K (few tiles, long K; only without a batch): grid z is the slice, every slice covers split_slabs slabs of K and
      leaves its raw sums in partial[z] (dense M x N planes, complex: real plane then imaginary plane); gemm_split_finish
      adds the slices in order and applies alpha / beta */
   uint32_t split_slabs;
   R       *partial;
};

#define OCH_GEMM_THREADS 256

/* Column twist of the k-major LDS planes. The row pitch moves every k on by 8 banks (of 32), so rows k and k + 4 start in
   the same bank; an operand that is contiguous along k in memory is stored by lanes that hold different k for the same
   column, and those stores collided (SQ_LDS_BANK_CONFLICT was a third to a half of the LDS cycles with such an operand,
   zero without). Element (k, c) therefore sits in column c ^ twist(k), twist = ((k / 4) mod 4) * (columns that the lanes of
   one LDS cycle cover): a multiple of the vector length and smaller than an MFMA tile, so vector stores along the row and
   the fragment reads of an aligned tile keep their shape. */
template <class R, bool CPLX, int KT> __device__ __forceinline__ uint32_t lds_twist(uint32_t k)
{  constexpr int VE = 16 / ((int)sizeof(R) * (CPLX ? 2 : 1));          /* elements per 128-bit load */
   constexpr int LANES = (sizeof(R) == 4) ? 32 : 16;                    /* lanes served per LDS cycle (128 bytes) */
   constexpr int COLS = LANES / (KT / VE);                              /* columns they cover when k varies fastest */
   return ((k >> 2) & 3u) * COLS;
}

/* Moves a BMN x KT slab of an operand from global memory to registers (fetch) and from there
   to its k-major LDS planes (stash). KC: the operand is contiguous along k in memory. */
template <class R, bool CPLX, bool KC, bool EDGE, int BMN, int KT>
struct SlabLoader
{
   static constexpr int NPL = CPLX ? 2 : 1;
   static constexpr int ES = (int)sizeof(R) * NPL;
   static constexpr int VE = 16 / ES;                              /* elements per 128-bit load */
   static constexpr int NV = BMN * KT / VE / OCH_GEMM_THREADS;     /* loads per thread */
   static_assert(NV >= 1 && (BMN * KT) % (VE * OCH_GEMM_THREADS) == 0, "slab does not divide among the threads");
   R reg[NV][VE * NPL];

   static __device__ __forceinline__ void where(int v, uint32_t &mn, uint32_t &k)
   {  const uint32_t q = threadIdx.x + OCH_GEMM_THREADS * v;
      if (!KC) { mn = (q % (BMN / VE)) * VE; k = q / (BMN / VE); }
      else     { k = (q % (KT / VE)) * VE;   mn = q / (KT / VE); }
   }
   /* mat: operand origin; element (mn, k) of op(.) lives at mn + k * ld (!KC) or k + mn * ld (KC) */
   __device__ __forceinline__ void fetch(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0, uint32_t MN, uint32_t K, int aligned)
   {
      /* Edge-handling kernel: a 128-bit vector that lies inside the matrix and is aligned is still one load (most vectors
         of most tiles), one that lies outside is zero without touching memory; only vectors that straddle the border, and
         all of them when the operand is not aligned, are loaded element by element. */
#pragma unroll
      for (int v = 0; v < NV; v++)
      {  uint32_t mn, k; where(v, mn, k);
         const int64_t gm = (int64_t)mn0 + mn, gk = (int64_t)k0 + k;
         const char *addr = mat + (KC ? (gk + gm * ld) : (gm + gk * ld)) * ES;
         bool whole = true;
         if (EDGE) whole = aligned && (KC ? (gm < (int64_t)MN && gk + VE <= (int64_t)K) : (gk < (int64_t)K && gm + VE <= (int64_t)MN));
         if (whole)
         {  och_gu32x4 raw = *reinterpret_cast<const och_gu32x4 *>(addr);
            __builtin_memcpy(&reg[v][0], &raw, 16);
         }
         else
         {
#pragma unroll
            for (int e = 0; e < VE; e++)
            {  const int64_t em = gm + (KC ? 0 : e), ek = gk + (KC ? e : 0);
               const bool ok = (em < (int64_t)MN) && (ek < (int64_t)K);
               const R *src = reinterpret_cast<const R *>(addr + (int64_t)e * ES);
#pragma unroll
               for (int c = 0; c < NPL; c++) reg[v][e * NPL + c] = ok ? src[c] : (R)0;
            }
         }
      }
   }
   /* planes: plane 0 of this operand in the current LDS buffer; row pitch in reals */
   __device__ __forceinline__ void stash(R *planes, int pitch, bool conj) const
   {
#pragma unroll
      for (int v = 0; v < NV; v++)
      {  uint32_t mn, k; where(v, mn, k);
#pragma unroll
         for (int e = 0; e < VE; e++)
         {  const uint32_t ek = k + (KC ? e : 0), em = (mn ^ lds_twist<R, CPLX, KT>(ek)) + (KC ? 0 : e);
            planes[ek * pitch + em] = reg[v][e * NPL];
            if (CPLX) planes[(KT + ek) * pitch + em] = conj ? -reg[v][e * NPL + 1] : reg[v][e * NPL + 1];
         }
      }
   }
};

template <class R, bool CPLX, bool AKC, bool BKC, bool EDGE, int WM, int WN, int KT>
__global__ __launch_bounds__(OCH_GEMM_THREADS, 2) void gemm_mfma_kernel(const GemmParams<R> p)
{
   typedef Mfma<R> MM;
   typedef typename MM::Acc Acc;
   constexpr int T = MM::T, TK = MM::TK;
   constexpr int BM = 2 * WM, BN = 2 * WN, NPL = CPLX ? 2 : 1;
   constexpr int TMS = WM / T, TNS = WN / T;
   constexpr int PAD = 32 / (int)sizeof(R);
   constexpr int PA = BM + PAD, PB = BN + PAD;
   constexpr int BUF = NPL * KT * (PA + PB);
   __shared__ __align__(16) R lds[2 * BUF];

   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const char *pA = p.A + oA, *pB = p.B + oB; char *pC = p.C + oC;
   const uint32_t tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
   const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   const int wm = (wave & 1) * WM, wn = (wave >> 1) * WN;

   Acc acc[TMS][TNS], acci[CPLX ? TMS : 1][CPLX ? TNS : 1];
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {
#pragma unroll
         for (int r = 0; r < MM::NACC; r++) { acc[i][j][r] = 0; if (CPLX) acci[i][j][r] = 0; }
      }

   SlabLoader<R, CPLX, AKC, EDGE, BM, KT> la;
   SlabLoader<R, CPLX, BKC, EDGE, BN, KT> lb;
   uint32_t slab0 = 0, nslabs = (p.K + KT - 1) / KT;
   if (p.split_slabs)
   {  slab0 = blockIdx.z * p.split_slabs;
      nslabs = (slab0 + p.split_slabs < nslabs) ? p.split_slabs : (slab0 < nslabs ? nslabs - slab0 : 0);
   }
   /* 4-byte reals (DEEP): registers hold the slab after the one in LDS; slab s + 1 is stored half way through the MFMAs of
      slab s and the loads of slab s + 2 are issued right after, a slab and a half before their data is needed (8192^3
      float: 121 / 124 / 131 -> 126 / 130 / 132 TFLOP/s for NN / TN / NT). For double, whose slab is two MFMA steps, the
      loads of slab s + 1 at the top of the iteration and its stores at the end measure better (66.5 against 64.0). */
   constexpr bool DEEP = (sizeof(R) == 4);
   if (nslabs > 0)
   {  la.fetch(pA, p.ldA, m0, slab0 * KT, p.M, p.K, p.alignedA);
      lb.fetch(pB, p.ldB, n0, slab0 * KT, p.N, p.K, p.alignedB);
      la.stash(lds, PA, p.conjA);
      lb.stash(lds + NPL * KT * PA, PB, p.conjB);
      if (DEEP && nslabs > 1)
      {  la.fetch(pA, p.ldA, m0, (slab0 + 1) * KT, p.M, p.K, p.alignedA);
         lb.fetch(pB, p.ldB, n0, (slab0 + 1) * KT, p.N, p.K, p.alignedB);
      }
   }
   __syncthreads();
   for (uint32_t s = 0; s < nslabs; s++)
   {  const R *As = lds + (s & 1) * BUF, *Bs = As + NPL * KT * PA;
      if (!DEEP && s + 1 < nslabs)
      {  la.fetch(pA, p.ldA, m0, (slab0 + s + 1) * KT, p.M, p.K, p.alignedA);
         lb.fetch(pB, p.ldB, n0, (slab0 + s + 1) * KT, p.N, p.K, p.alignedB);
      }
#pragma unroll
      for (int ks = 0; ks < KT / TK; ks++)
      {  const int k = ks * TK + lane / T;
         R a[TMS], b[TNS], ai[CPLX ? TMS : 1], bi[CPLX ? TNS : 1];
#pragma unroll
         for (int i = 0; i < TMS; i++)
         {  a[i] = As[k * PA + ((wm + i * T + lane % T) ^ lds_twist<R, CPLX, KT>(k))];
            if (CPLX) ai[i] = As[(KT + k) * PA + ((wm + i * T + lane % T) ^ lds_twist<R, CPLX, KT>(k))];
         }
#pragma unroll
         for (int j = 0; j < TNS; j++)
         {  b[j] = Bs[k * PB + ((wn + j * T + lane % T) ^ lds_twist<R, CPLX, KT>(k))];
            if (CPLX) bi[j] = Bs[(KT + k) * PB + ((wn + j * T + lane % T) ^ lds_twist<R, CPLX, KT>(k))];
         }
#pragma unroll
         for (int i = 0; i < TMS; i++)
#pragma unroll
            for (int j = 0; j < TNS; j++)
            {  acc[i][j] = MM::mma(a[i], b[j], acc[i][j]);
               if (CPLX)
               {  acc[i][j]  = MM::mma(-ai[i], bi[j], acc[i][j]);
                  acci[i][j] = MM::mma(a[i], bi[j], acci[i][j]);
                  acci[i][j] = MM::mma(ai[i], b[j], acci[i][j]);
               }
            }
         if (DEEP && ks == (KT / TK) / 2 - 1 && s + 1 < nslabs)
         {  R *An = lds + ((s + 1) & 1) * BUF;
            la.stash(An, PA, p.conjA);
            lb.stash(An + NPL * KT * PA, PB, p.conjB);
            if (s + 2 < nslabs)
            {  la.fetch(pA, p.ldA, m0, (slab0 + s + 2) * KT, p.M, p.K, p.alignedA);
               lb.fetch(pB, p.ldB, n0, (slab0 + s + 2) * KT, p.N, p.K, p.alignedB);
            }
         }
      }
      if (!DEEP && s + 1 < nslabs)
      {  R *An = lds + ((s + 1) & 1) * BUF;
         la.stash(An, PA, p.conjA);
         lb.stash(An + NPL * KT * PA, PB, p.conjB);
      }
      __syncthreads();
   }

   if (p.split_slabs)
   {  /* raw sums of this K slice */
      R *plane = p.partial + (size_t)blockIdx.z * NPL * p.M * p.N;
#pragma unroll
      for (int i = 0; i < TMS; i++)
#pragma unroll
         for (int j = 0; j < TNS; j++)
         {  const uint32_t col = n0 + wn + j * T + lane % T;
#pragma unroll
            for (int r = 0; r < MM::NACC; r++)
            {  const uint32_t row = m0 + wm + i * T + MM::acc_row(lane, r);
               if (row >= p.M || col >= p.N) continue;
               plane[(size_t)col * p.M + row] = acc[i][j][r];
               if (CPLX) plane[(size_t)p.M * p.N + (size_t)col * p.M + row] = acci[i][j][r];
            }
         }
      return;
   }

   /* epilogue */
   R alr = p.alpha[0], ali = p.alpha[1], ber = p.beta[0], bei = p.beta[1];
   if (p.alpha_dev) { const R *q = reinterpret_cast<const R *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha); alr = q[0]; if (CPLX) ali = q[1]; }
   if (p.beta_dev)  { const R *q = reinterpret_cast<const R *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);   ber = q[0]; if (CPLX) bei = q[1]; }
   const bool use_c = CPLX ? (ber != 0 || bei != 0) : (ber != 0);
#pragma unroll
   for (int i = 0; i < TMS; i++)
#pragma unroll
      for (int j = 0; j < TNS; j++)
      {  const uint32_t col = n0 + wn + j * T + lane % T;
#pragma unroll
         for (int r = 0; r < MM::NACC; r++)
         {  const uint32_t row = m0 + wm + i * T + MM::acc_row(lane, r);
            if (EDGE && (row >= p.M || col >= p.N)) continue;
            R *c = reinterpret_cast<R *>(pC + ((int64_t)row + (int64_t)col * p.ldC) * (int64_t)(sizeof(R) * NPL));
            if (!CPLX)
            {  R v = alr * acc[i][j][r];
               if (use_c) v += ber * c[0];
               c[0] = v;
            }
            else
            {  const R sr = acc[i][j][r], si = acci[i][j][r];
               R vr = alr * sr - ali * si, vi = alr * si + ali * sr;
               if (use_c) { const R cr = c[0], ci = c[1]; vr += ber * cr - bei * ci; vi += ber * ci + bei * cr; }
               c[0] = vr; c[1] = vi;
            }
         }
      }
}

/* adds the K slices of a split product in slice order and applies alpha / beta: one thread per element of C */
template <class R, bool CPLX>
__global__ __launch_bounds__(256) void gemm_split_finish_kernel(const GemmParams<R> p, uint32_t slices)
{
   constexpr int NPL = CPLX ? 2 : 1;
   const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x, mn = (uint64_t)p.M * p.N;
   if (e >= mn) return;
   const uint32_t col = (uint32_t)(e / p.M), row = (uint32_t)(e - (uint64_t)col * p.M);
   R sr = 0, si = 0;
   uint32_t t = 0;
   for (; t + 7 < slices; t += 8)
   {  R vr[8], vi[8];
#pragma unroll
      for (int u = 0; u < 8; u++) { vr[u] = p.partial[(size_t)(t + u) * NPL * mn + e]; if (CPLX) vi[u] = p.partial[(size_t)(t + u) * NPL * mn + mn + e]; }
#pragma unroll
      for (int u = 0; u < 8; u++) { sr += vr[u]; if (CPLX) si += vi[u]; }
   }
   for (; t < slices; t++) { sr += p.partial[(size_t)t * NPL * mn + e]; if (CPLX) si += p.partial[(size_t)t * NPL * mn + mn + e]; }
   R alr = p.alpha[0], ali = p.alpha[1], ber = p.beta[0], bei = p.beta[1];
   if (p.alpha_dev) { alr = p.alpha_dev[0]; if (CPLX) ali = p.alpha_dev[1]; }
   if (p.beta_dev)  { ber = p.beta_dev[0];  if (CPLX) bei = p.beta_dev[1]; }
   R *c = reinterpret_cast<R *>(p.C) + ((int64_t)row + (int64_t)col * p.ldC) * NPL;
   if (!CPLX)
   {  R v = alr * sr;
      if (ber != 0) v += ber * c[0];
      c[0] = v;
   }
   else
   {  R vr = alr * sr - ali * si, vi = alr * si + ali * sr;
      if (ber != 0 || bei != 0) { const R cr = c[0], ci = c[1]; vr += ber * cr - bei * ci; vi += ber * ci + bei * cr; }
      c[0] = vr; c[1] = vi;
   }
}

/* Few outputs (dot products, tiny C): one block per element of C strides over K. Accumulates
   in double; the four partial sums of the waves are folded in wave order. */
template <class R, bool CPLX>
__global__ __launch_bounds__(256) void gemm_dot_kernel(const GemmParams<R> p, int64_t sAm, int64_t sAk, int64_t sBk, int64_t sBn)
{
   constexpr int NPL = CPLX ? 2 : 1;
   __shared__ double lds[8];
   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const uint32_t row = blockIdx.x % p.M, col = blockIdx.x / p.M;
   const R *a = reinterpret_cast<const R *>(p.A + oA) + (int64_t)row * sAm * NPL;
   const R *b = reinterpret_cast<const R *>(p.B + oB) + (int64_t)col * sBn * NPL;
   double sr = 0, si = 0;
   if (!CPLX)
   {  /* four independent loads and partial sums per trip: the block is alone on its compute unit and latency-bound */
      double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
      uint32_t k = threadIdx.x;
      for (; k + 768 < p.K; k += 1024)
      {  const R x0 = a[(int64_t)k * sAk], x1 = a[(int64_t)(k + 256) * sAk], x2 = a[(int64_t)(k + 512) * sAk], x3 = a[(int64_t)(k + 768) * sAk];
         const R y0 = b[(int64_t)k * sBk], y1 = b[(int64_t)(k + 256) * sBk], y2 = b[(int64_t)(k + 512) * sBk], y3 = b[(int64_t)(k + 768) * sBk];
         s0 += (double)x0 * (double)y0; s1 += (double)x1 * (double)y1; s2 += (double)x2 * (double)y2; s3 += (double)x3 * (double)y3;
      }
      for (; k < p.K; k += 256) s0 += (double)a[(int64_t)k * sAk] * (double)b[(int64_t)k * sBk];
      sr = (s0 + s1) + (s2 + s3);
   }
   else
   {  for (uint32_t k = threadIdx.x; k < p.K; k += 256)
      {  const R *x = a + (int64_t)k * sAk * NPL, *y = b + (int64_t)k * sBk * NPL;
         const double xr = x[0], xi = p.conjA ? -(double)x[1] : (double)x[1];
         const double yr = y[0], yi = p.conjB ? -(double)y[1] : (double)y[1];
         sr += xr * yr - xi * yi; si += xr * yi + xi * yr;
      }
   }
#pragma unroll
   for (int m = 32; m >= 1; m >>= 1) { sr += __shfl_xor(sr, m, 64); if (CPLX) si += __shfl_xor(si, m, 64); }
   if ((threadIdx.x & 63) == 0) { lds[(threadIdx.x >> 6) * 2] = sr; lds[(threadIdx.x >> 6) * 2 + 1] = si; }
   __syncthreads();
   if (threadIdx.x != 0) return;
   sr = ((lds[0] + lds[2]) + lds[4]) + lds[6];
   si = ((lds[1] + lds[3]) + lds[5]) + lds[7];
   R alr = p.alpha[0], ali = p.alpha[1], ber = p.beta[0], bei = p.beta[1];
   if (p.alpha_dev) { const R *q = reinterpret_cast<const R *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha); alr = q[0]; if (CPLX) ali = q[1]; }
   if (p.beta_dev)  { const R *q = reinterpret_cast<const R *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);   ber = q[0]; if (CPLX) bei = q[1]; }
   R *c = reinterpret_cast<R *>(p.C + oC) + ((int64_t)row + (int64_t)col * p.ldC) * NPL;
   if (!CPLX)
   {  double v = (double)alr * sr;
      if (ber != 0) v += (double)ber * (double)c[0];
      c[0] = (R)v;
   }
   else
   {  double vr = (double)alr * sr - (double)ali * si, vi = (double)alr * si + (double)ali * sr;
      if (ber != 0 || bei != 0)
      {  const double cr = c[0], ci = c[1];
         vr += (double)ber * cr - (double)bei * ci; vi += (double)ber * ci + (double)bei * cr;
      }
      c[0] = (R)vr; c[1] = (R)vi;
   }
}

/* Very short inner dimension (rank-1 updates, K <= 4): one thread per element of C reads its K products directly;
   the tile machinery of the MFMA kernel would spend its time on padding. Accumulates in double. */
template <class R, bool CPLX>
__global__ __launch_bounds__(256) void gemm_outer_kernel(const GemmParams<R> p, int64_t sAm, int64_t sAk, int64_t sBk, int64_t sBn)
{
   constexpr int NPL = CPLX ? 2 : 1;
   int64_t oA, oB, oC, oAlpha, oBeta;
   gemm_batch_offsets(p.batch, oA, oB, oC, oAlpha, oBeta);
   const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
   if (e >= (uint64_t)p.M * p.N) return;
   const uint32_t col = (uint32_t)(e / p.M), row = (uint32_t)(e - (uint64_t)col * p.M);
   const R *a = reinterpret_cast<const R *>(p.A + oA) + (int64_t)row * sAm * NPL;
   const R *b = reinterpret_cast<const R *>(p.B + oB) + (int64_t)col * sBn * NPL;
   double sr = 0, si = 0;
   for (uint32_t k = 0; k < p.K; k++)
   {  const R *x = a + (int64_t)k * sAk * NPL, *y = b + (int64_t)k * sBk * NPL;
      if (!CPLX) sr += (double)x[0] * (double)y[0];
      else
      {  const double xr = x[0], xi = p.conjA ? -(double)x[1] : (double)x[1];
         const double yr = y[0], yi = p.conjB ? -(double)y[1] : (double)y[1];
         sr += xr * yr - xi * yi; si += xr * yi + xi * yr;
      }
   }
   R alr = p.alpha[0], ali = p.alpha[1], ber = p.beta[0], bei = p.beta[1];
   if (p.alpha_dev) { const R *q = reinterpret_cast<const R *>(reinterpret_cast<const char *>(p.alpha_dev) + oAlpha); alr = q[0]; if (CPLX) ali = q[1]; }
   if (p.beta_dev)  { const R *q = reinterpret_cast<const R *>(reinterpret_cast<const char *>(p.beta_dev) + oBeta);   ber = q[0]; if (CPLX) bei = q[1]; }
   R *c = reinterpret_cast<R *>(p.C + oC) + ((int64_t)row + (int64_t)col * p.ldC) * NPL;
   if (!CPLX)
   {  double v = (double)alr * sr;
      if (ber != 0) v += (double)ber * (double)c[0];
      c[0] = (R)v;
   }
   else
   {  double vr = (double)alr * sr - (double)ali * si, vi = (double)alr * si + (double)ali * sr;
      if (ber != 0 || bei != 0)
      {  const double cr = c[0], ci = c[1];
         vr += (double)ber * cr - (double)bei * ci; vi += (double)ber * ci + (double)bei * cr;
      }
      c[0] = (R)vr; c[1] = (R)vi;
   }
}

/* host side ------------------------------------------------------------------ */
struct GemmArgs
{
   char transA, transB;
   size_t M, N, K;
   const void *alpha, *beta;
   const void *A, *B; void *C;
   ptrdiff_t ldA, ldB, ldC;
   int scalar_mode_host;
   hipStream_t stream;
   GemmBatch batch;                 /* nb = 0: one product */
   unsigned  nz;                    /* grid z: batch entries of this launch (1 when nb = 0) */
};

template <class R, bool CPLX, int WM, int WN, int KT>
static int launch_gemm_mfma(const GemmArgs &g)
{
   constexpr int NPL = CPLX ? 2 : 1;
   constexpr int ES = (int)sizeof(R) * NPL;
   constexpr int BM = 2 * WM, BN = 2 * WN;
   GemmParams<R> p;
   memset(&p, 0, sizeof(p));
   p.A = (const char *)g.A; p.B = (const char *)g.B; p.C = (char *)g.C;
   p.ldA = g.ldA; p.ldB = g.ldB; p.ldC = g.ldC;
   p.M = (uint32_t)g.M; p.N = (uint32_t)g.N; p.K = (uint32_t)g.K;
   if (g.scalar_mode_host)
   {  memcpy(p.alpha, g.alpha, ES); memcpy(p.beta, g.beta, ES); }
   else
   {  p.alpha_dev = (const R *)g.alpha; p.beta_dev = (const R *)g.beta; }
   p.batch = g.batch;
   const bool akc = (g.transA != 'N'), bkc = (g.transB == 'N');
   p.conjA = CPLX && (g.transA == 'C'); p.conjB = CPLX && (g.transB == 'C');

   if (g.M * g.N <= 256 && g.K >= 64)
   {  /* op(A)(m,k) = A[m*sAm + k*sAk], op(B)(k,n) = B[k*sBk + n*sBn] */
      const int64_t sAm = akc ? g.ldA : 1, sAk = akc ? 1 : g.ldA, sBk = bkc ? 1 : g.ldB, sBn = bkc ? g.ldB : 1;
      hipLaunchKernelGGL((gemm_dot_kernel<R, CPLX>), dim3((unsigned)(g.M * g.N), 1, g.nz), dim3(256), 0, g.stream, p, sAm, sAk, sBk, sBn);
      OCH_CHECK_LAUNCH();
      return 0;
   }
   if (g.K <= 4 && (uint64_t)g.M * g.N <= 0x7FFFFFFFull * 256)
   {  const int64_t sAm = akc ? g.ldA : 1, sAk = akc ? 1 : g.ldA, sBk = bkc ? 1 : g.ldB, sBn = bkc ? g.ldB : 1;
      hipLaunchKernelGGL((gemm_outer_kernel<R, CPLX>), dim3((unsigned)(((uint64_t)g.M * g.N + 255) / 256), 1, g.nz), dim3(256), 0, g.stream, p, sAm, sAk, sBk, sBn);
      OCH_CHECK_LAUNCH();
      return 0;
   }
   if (g.batch.nb == 0 && (g.N <= OCH_GEMV_MAX_S || g.M <= OCH_GEMV_MAX_S) && (g.M >= 64 || g.N >= 64))
   {  /* one very small dimension: stream the large operand once (och_gemv.h) */
      const int64_t sAm = akc ? g.ldA : 1, sAk = akc ? 1 : g.ldA, sBk = bkc ? 1 : g.ldB, sBn = bkc ? g.ldB : 1;
      GemvParams<R> v;
      memset(&v, 0, sizeof(v));
      if (g.N <= g.M)
      {  v.X = (const R *)g.A; v.sXr = sAm; v.sXk = sAk; v.conjX = p.conjA; v.Y = (const R *)g.B; v.sYk = sBk; v.sYs = sBn; v.conjY = p.conjB;
         v.O = (R *)g.C; v.sOr = 1; v.sOs = g.ldC; v.rows = (uint32_t)g.M; v.S = (uint32_t)g.N;
      }
      else
      {  v.X = (const R *)g.B; v.sXr = sBn; v.sXk = sBk; v.conjX = p.conjB; v.Y = (const R *)g.A; v.sYk = sAk; v.sYs = sAm; v.conjY = p.conjA;
         v.O = (R *)g.C; v.sOr = g.ldC; v.sOs = 1; v.rows = (uint32_t)g.N; v.S = (uint32_t)g.M;
      }
      v.K = (uint32_t)g.K;
      memcpy(v.alpha, p.alpha, sizeof(v.alpha)); memcpy(v.beta, p.beta, sizeof(v.beta));
      v.alpha_dev = p.alpha_dev; v.beta_dev = p.beta_dev;
      const int status = launch_gemv<R, CPLX>(v, g.stream);
      if (status != 0) return status < 0 ? -1 : 0;
   }
   p.tiles_m = (uint32_t)((g.M + BM - 1) / BM); p.tiles_n = (uint32_t)((g.N + BN - 1) / BN);
   const uint64_t blocks = (uint64_t)p.tiles_m * p.tiles_n;
   if (blocks > 0x7FFFFFFFull) return set_error("gemm: too many tiles");
   auto aligned = [&](const void *ptr, ptrdiff_t ld, const int64_t *bs)
   {  bool ok = ((uintptr_t)ptr % 16 == 0) && (((int64_t)ld * ES) % 16 == 0);
      for (int d = 0; d < g.batch.nb; d++) ok = ok && (bs[d] % 16 == 0);                 /* every batch entry */
      return ok;
   };
   p.alignedA = aligned(g.A, g.ldA, g.batch.sA) ? 1 : 0; p.alignedB = aligned(g.B, g.ldB, g.batch.sB) ? 1 : 0;
   const bool edge = !(g.M % BM == 0 && g.N % BN == 0 && g.K % KT == 0 && p.alignedA && p.alignedB);
   /* few tiles and a long K: slices of K in grid z, at least 16 slabs each, about 512 blocks in all, partial sums within the workspace */
   uint32_t slices = 1;
   {  const uint64_t nslabs = (g.K + KT - 1) / KT;
      if (g.batch.nb == 0 && blocks < 128 && nslabs >= 64)
      {  uint64_t want = (512 + blocks - 1) / blocks;
         if (want > nslabs / 16) want = nslabs / 16;
         const uint64_t fit = OCH_GEMM_WORKSPACE / ((uint64_t)g.M * g.N * ES);
         if (want > fit) want = fit;
         if (want > 65535) want = 65535;
         if (want >= 2)
         {  char *ws;
            if (stream_gemm_workspace(g.stream, &ws) != 0) return -1;
            p.split_slabs = (uint32_t)((nslabs + want - 1) / want);
            slices = (uint32_t)((nslabs + p.split_slabs - 1) / p.split_slabs);
            p.partial = reinterpret_cast<R *>(ws);
            if (slices < 2) { slices = 1; p.split_slabs = 0; p.partial = nullptr; }
         }
      }
   }
   const dim3 grid((unsigned)blocks, 1, slices > 1 ? slices : g.nz), block(OCH_GEMM_THREADS);
#define OCH_GEMM_LAUNCH(AK, BK)                                                                             \
   do { if (edge) hipLaunchKernelGGL((gemm_mfma_kernel<R, CPLX, AK, BK, true, WM, WN, KT>), grid, block, 0, g.stream, p);  \
        else      hipLaunchKernelGGL((gemm_mfma_kernel<R, CPLX, AK, BK, false, WM, WN, KT>), grid, block, 0, g.stream, p); } while (0)
   if (!akc && !bkc) OCH_GEMM_LAUNCH(false, false);
   else if (!akc)    OCH_GEMM_LAUNCH(false, true);
   else if (!bkc)    OCH_GEMM_LAUNCH(true, false);
   else              OCH_GEMM_LAUNCH(true, true);
#undef OCH_GEMM_LAUNCH
   if (slices > 1)
      hipLaunchKernelGGL((gemm_split_finish_kernel<R, CPLX>), dim3((unsigned)(((uint64_t)g.M * g.N + 255) / 256)), dim3(256), 0, g.stream, p, slices);
   OCH_CHECK_LAUNCH();
   return 0;
}

/* one load from memory straight to LDS: lane l brings 16 bytes from base + offset[l] to LDS byte target + 16 l. The target
   travels in M0, which the kernels that load this way use for nothing else (the compiler is not told: it counts M0 among the registers it
   manages itself and warns about a clobber); the compiler does not see a load either, so the waits for these loads
   (vmcnt) are written out in front of the barriers. */
static __device__ __forceinline__ void load_to_lds(const char *base, uint32_t offset, uint32_t target)
{
   asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(target), "v"(offset), "s"(base) : "memory");
}

/* Compute units of the current device (cached per device). */
int gemm_compute_units(void);
int gemm_kernel_choice(void);            /* 0 automatic; 1 / 2 / 4: pipelined kernel, large / small / smallest tile; 3: never pipelined */
int gemm_pipe_split_plan(uint64_t M, uint64_t N, uint64_t K, uint64_t batch, bool single, uint32_t tile_m, uint32_t tile_n,
                         uint32_t slab, uint32_t elem_size, uint64_t units, double *rounds);   /* shares of the tiles of the last round */
int gemm_pad_tail(const GemmArgs &g, size_t Kh, int slab, int es, GemmArgs *tail);   /* the rest of K as one zero-padded slab in the workspace */

/* A product on a pipelined kernel whose K need not be a whole number of slabs (the caller has checked that the scalars
   are in host memory when it is not): the whole slabs through `pipelined` with the caller's beta, then the rest of K --
   both operands' tails copied into the workspace and filled up with zeros to one slab -- through `pipelined` again with
   beta = 1 (`one`: that scalar in the product's type); where the rest cannot be padded, through `others`, the type's own
   entry. 0: done; 1: the pipelined kernel does not take the product, nothing was launched; -1: error. es: element size. */
template <class Pipelined, class Others>
static int gemm_pipelined_head_and_rest(const GemmArgs &g, int slab, int es, const void *one, Pipelined pipelined, Others others)
{
   GemmArgs part = g;
   const size_t Kh = g.K - g.K % (size_t)slab;
   part.K = Kh;
   const int taken = pipelined(part);
   if (taken != 0) return taken;
   if (g.K == Kh) return 0;
   GemmArgs tail;
   const int padded = gemm_pad_tail(g, Kh, slab, es, &tail);
   if (padded < 0) return -1;
   if (padded == 0)
   {  tail.beta = one;
      const int again = pipelined(tail);
      if (again < 0) return -1;
      if (again == 0) return 0;
   }
   part.K = g.K - Kh; part.beta = one;
   part.A = (const char *)g.A + (int64_t)Kh * (g.transA == 'N' ? (int64_t)g.ldA : 1) * es;
   part.B = (const char *)g.B + (int64_t)Kh * (g.transB == 'N' ? 1 : (int64_t)g.ldB) * es;
   return others(part) != 0 ? -1 : 0;
}

/* Which block tile to use. The compute units work through the tiles in rounds, and the last round is as long as the others
   however few tiles it holds: 3000^3 double is 576 tiles of 128 x 128, i.e. 2.25 rounds on 256 units, and ran at 39
   TFLOP/s where 4000^3 (exactly 4 rounds) reached 56. A candidate's cost is rounds x tile area / efficiency (its measured
   efficiency on large products, relative to the largest tile): the time the product takes in units of one element of C
   per compute unit. It also charges the part of edge tiles that lies outside C, so a dot product does not get the
   largest tile. The cheapest candidate wins; within 2 % the larger tile (earlier in the list) is kept. */
struct GemmTileChoice { int bm, bn; double efficiency; };
static inline int gemm_pick_tile(const GemmArgs &g, const GemmTileChoice *choice, int n)
{  if ((g.M * g.N <= 256 && g.K >= 64) || g.K <= 4) return n - 1;       /* dot and outer products have kernels of their own: no tile to choose */
   const uint64_t units = (uint64_t)gemm_compute_units();
   int best = 0; double best_cost = 0;
   for (int c = 0; c < n; c++)
   {  const uint64_t tiles = ((g.M + choice[c].bm - 1) / choice[c].bm) * ((g.N + choice[c].bn - 1) / choice[c].bn) * (uint64_t)g.nz;
      const uint64_t rounds = (tiles + units - 1) / units;
      const double cost = (double)rounds * choice[c].bm * choice[c].bn / choice[c].efficiency;
      if (c == 0 || cost < best_cost * 0.98) { best = c; best_cost = cost; }
   }
   return best;
}

/* base pointers, leading dimensions and batch strides of all three operands allow 16-byte accesses (es: element size) */
static inline bool gemm_operands_aligned(const GemmArgs &g, int es)
{  bool ok = ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) && ((uintptr_t)g.C % 16 == 0)
          && ((int64_t)g.ldA * es) % 16 == 0 && ((int64_t)g.ldB * es) % 16 == 0 && ((int64_t)g.ldC * es) % 16 == 0;
   for (int d = 0; d < g.batch.nb; d++) ok = ok && g.batch.sA[d] % 16 == 0 && g.batch.sB[d] % 16 == 0 && g.batch.sC[d] % 16 == 0;
   return ok;
}

int gemm_float(const GemmArgs &g);
int gemm_float_pipe(const GemmArgs &g, int tile); /* tiles of 256 x 256, 128 x 128 or 64 x 64; 1: not taken */
int gemm_float_plan_query(uint64_t M, uint64_t N, uint64_t K, unsigned batch); /* the tile an aligned product takes; 0: the tiled kernels */
int gemm_float_pipe_split(const GemmArgs &g, int tile, double *rounds); /* shares of the tiles of the last round; rounds of the compute units */
int gemm_double(const GemmArgs &g);
int gemm_double_pipe(const GemmArgs &g, int tile_m); /* tiles of 256 x 128 or 128 x 128; 1: not taken */
int gemm_double_pipe_split(const GemmArgs &g, int tile_m, double *rounds); /* shares of the tiles of the last round; rounds of the compute units */
int gemm_cfloat(const GemmArgs &g);
int gemm_cfloat_pipe(const GemmArgs &g); /* tiles of 128 x 128; 1: not taken */
int gemm_cfloat_pipe_split(const GemmArgs &g, double *rounds);
int gemm_cdouble(const GemmArgs &g);
int gemm_cdouble_pipe(const GemmArgs &g); /* tiles of 128 x 64; 1: not taken */
int gemm_cdouble_pipe_split(const GemmArgs &g, double *rounds);
int gemm_half(const GemmArgs &g);      /* 1: not taken, use the generic kernel */
int gemm_int8(const GemmArgs &g);      /* int8 and uint8; 1: not taken */
int gemm_bool(const GemmArgs &g);      /* 1: not taken */

} /* namespace och */
