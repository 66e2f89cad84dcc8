/* Matrix products with one very small dimension (matrix x vector, matrix x a few columns, and their transposes):
 * bandwidth-bound, so they stream the large operand once instead of going through the 128 x 128 MFMA tiles, which
 * would compute 127 of 128 columns for nothing (measured before: 8192 x 8192 times a vector 1.36 ms, the operand
 * itself streams in 0.09 ms).
 *
 * The product is written as O (rows x S) = X (rows x K) * Y (K x S), S <= 8, with element strides for every operand,
 * so that C = op(A) * op(B) with small N (X = op(A)) and with small M (X = op(B)^T, O = C^T) are the same code.
 *   gemv_rows_kernel: X is contiguous along the rows. A thread owns VEC neighbouring rows and walks a slice of K;
 *                     the K slices (grid y) leave double-precision partial results in the stream's workspace and
 *                     gemv_finish_kernel adds them in slice order (deterministic) and applies alpha / beta.
 *   gemv_dots_kernel: X is contiguous along K. 8-64 lanes share a row, each walks K with 128-bit loads; shuffle
 *                     reduction, no workspace.
 * Sums are accumulated in double for every type. */
#pragma once
#include "och_elemwise.h"

namespace och {

#define OCH_GEMV_MAX_S 8

template <class R> struct GemvParams
{
   const R *X, *Y; R *O;
   int64_t  sXr, sXk, sYk, sYs, sOr, sOs;     /* element strides (complex: in complex elements) */
   uint32_t rows, S, K;
   int      conjX, conjY;
   R        alpha[2], beta[2];
   const R *alpha_dev, *beta_dev;
   double  *partials;                         /* [slice][s][row] (complex: two planes per s) */
   uint32_t slices, kper;                     /* K slices and their length */
   uint32_t lanes;                            /* lanes per row in the dots kernel */
};

template <class R, bool CPLX> __device__ __forceinline__ void gemv_scalars(const GemvParams<R> &p, double &alr, double &ali, double &ber, double &bei)
{  alr = p.alpha[0]; ali = p.alpha[1]; ber = p.beta[0]; bei = p.beta[1];
   if (p.alpha_dev) { alr = p.alpha_dev[0]; ali = CPLX ? (double)p.alpha_dev[1] : 0.0; }
   if (p.beta_dev)  { ber = p.beta_dev[0];  bei = CPLX ? (double)p.beta_dev[1] : 0.0; }
}
template <class R, bool CPLX> __device__ __forceinline__ void gemv_store(const GemvParams<R> &p, uint32_t row, uint32_t s, double sr, double si,
                                                                        double alr, double ali, double ber, double bei)
{  constexpr int NPL = CPLX ? 2 : 1;
   R *o = p.O + ((int64_t)row * p.sOr + (int64_t)s * p.sOs) * NPL;
   if (!CPLX)
   {  double v = alr * sr;
      if (ber != 0) v += ber * (double)o[0];
      o[0] = (R)v;
   }
   else
   {  double vr = alr * sr - ali * si, vi = alr * si + ali * sr;
      if (ber != 0 || bei != 0) { const double cr = o[0], ci = o[1]; vr += ber * cr - bei * ci; vi += ber * ci + bei * cr; }
      o[0] = (R)vr; o[1] = (R)vi;
   }
}

/* X contiguous along the rows: thread = VEC rows, block = 256 * VEC rows, grid y = K slice */
template <class R, bool CPLX, int S, int VEC>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const GemvParams<R> p)
{
   constexpr int NPL = CPLX ? 2 : 1;
   const uint32_t r0 = (blockIdx.x * 256 + threadIdx.x) * VEC;
   if (r0 >= p.rows) return;
   const uint32_t k0 = blockIdx.y * p.kper, k1 = (k0 + p.kper < p.K) ? k0 + p.kper : p.K;
   double ar[S][VEC], ai[CPLX ? S : 1][CPLX ? VEC : 1];
#pragma unroll
   for (int s = 0; s < S; s++)
#pragma unroll
      for (int v = 0; v < VEC; v++) { ar[s][v] = 0; if (CPLX) ai[s][v] = 0; }
   const R *x = p.X + (int64_t)r0 * NPL;
   auto fetch = [&](Pack<R, VEC * NPL> &xv, uint32_t k)
   {  const R *xp = x + (int64_t)k * p.sXk * NPL;
      if (VEC * NPL > 1) load_wide<R, VEC * NPL, true>(xv, reinterpret_cast<const char *>(xp));
      else xv.v[0] = xp[0];
   };
   auto accumulate = [&](const Pack<R, VEC * NPL> &xv, uint32_t k)
   {
#pragma unroll
      for (int s = 0; s < S; s++)
      {  if (s < (int)p.S)
         {  const R *yp = p.Y + ((int64_t)k * p.sYk + (int64_t)s * p.sYs) * NPL;
            if (!CPLX)
            {  const double y = yp[0];
#pragma unroll
               for (int v = 0; v < VEC; v++) ar[s][v] += (double)xv.v[v] * y;
            }
            else
            {  const double yr = yp[0], yi = p.conjY ? -(double)yp[1] : (double)yp[1];
#pragma unroll
               for (int v = 0; v < VEC; v++)
               {  const double xr = xv.v[2 * v], xi = p.conjX ? -(double)xv.v[2 * v + 1] : (double)xv.v[2 * v + 1];
                  ar[s][v] += xr * yr - xi * yi; ai[s][v] += xr * yi + xi * yr;
               }
            }
         }
      }
   };
   uint32_t k = k0;
   for (; k + 7 < k1; k += 8)                            /* eight loads of the large operand in flight */
   {  Pack<R, VEC * NPL> xv[8];
#pragma unroll
      for (int u = 0; u < 8; u++) fetch(xv[u], k + u);
#pragma unroll
      for (int u = 0; u < 8; u++) accumulate(xv[u], k + u);
   }
   for (; k < k1; k++) { Pack<R, VEC * NPL> xv; fetch(xv, k); accumulate(xv, k); }
   if (p.slices == 1)
   {  double alr, ali, ber, bei;
      gemv_scalars<R, CPLX>(p, alr, ali, ber, bei);
#pragma unroll
      for (int s = 0; s < S; s++)
#pragma unroll
         for (int v = 0; v < VEC; v++) if (s < (int)p.S) gemv_store<R, CPLX>(p, r0 + v, s, ar[s][v], CPLX ? ai[s][v] : 0.0, alr, ali, ber, bei);
      return;
   }
#pragma unroll
   for (int s = 0; s < S; s++)
   {  if (s < (int)p.S)
      {  double *dst = p.partials + ((size_t)(blockIdx.y * p.S + s) * NPL) * p.rows + r0;
#pragma unroll
         for (int v = 0; v < VEC; v++) { dst[v] = ar[s][v]; if (CPLX) dst[p.rows + v] = ai[s][v]; }
      }
   }
}

/* adds the K slices in slice order and applies alpha / beta: one thread per element of O */
template <class R, bool CPLX>
__global__ __launch_bounds__(256) void gemv_finish_kernel(const GemvParams<R> p)
{
   constexpr int NPL = CPLX ? 2 : 1;
   const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
   if (e >= (uint64_t)p.rows * p.S) return;
   const uint32_t s = (uint32_t)(e / p.rows), row = (uint32_t)(e - (uint64_t)s * p.rows);
   double sr = 0, si = 0;
   const size_t step = (size_t)p.S * NPL * p.rows;                      /* from one slice to the next */
   const double *src = p.partials + ((size_t)s * NPL) * p.rows + row;
   uint32_t t = 0;
   for (; t + 7 < p.slices; t += 8)                                     /* loads first, then the sums in slice order */
   {  double vr[8], vi[8];
#pragma unroll
      for (int u = 0; u < 8; u++) { vr[u] = src[(t + u) * step]; if (CPLX) vi[u] = src[(t + u) * step + p.rows]; }
#pragma unroll
      for (int u = 0; u < 8; u++) { sr += vr[u]; if (CPLX) si += vi[u]; }
   }
   for (; t < p.slices; t++) { sr += src[t * step]; if (CPLX) si += src[t * step + p.rows]; }
   double alr, ali, ber, bei;
   gemv_scalars<R, CPLX>(p, alr, ali, ber, bei);
   gemv_store<R, CPLX>(p, row, s, sr, si, alr, ali, ber, bei);
}

/* X contiguous along K: p.lanes lanes per row (a power of two, 8 .. 64), VEC elements of K per lane and step */
template <class R, bool CPLX, int S, int VEC, bool YWIDE = false>
__global__ __launch_bounds__(256) void gemv_dots_kernel(const GemvParams<R> p)
{
   constexpr int NPL = CPLX ? 2 : 1;
   const uint32_t G = p.lanes, lane = threadIdx.x % G;
   const uint32_t row = blockIdx.x * (256 / G) + threadIdx.x / G;
   const bool active = row < p.rows;
   double ar[S], ai[CPLX ? S : 1];
#pragma unroll
   for (int s = 0; s < S; s++) { ar[s] = 0; if (CPLX) ai[s] = 0; }
   if (active)
   {  const R *x = p.X + (int64_t)row * p.sXr * NPL;
      const uint32_t kfull = p.K - p.K % VEC;
      auto fetch = [&](Pack<R, VEC * NPL> &xv, uint32_t k)
      {  if (VEC * NPL > 1) load_wide<R, VEC * NPL, true>(xv, reinterpret_cast<const char *>(x + (int64_t)k * NPL));
         else xv.v[0] = x[k];
      };
      auto accumulate = [&](const Pack<R, VEC * NPL> &xv, uint32_t k)
      {
#pragma unroll
         for (int s = 0; s < S; s++)
         {  if (s < (int)p.S)
            {  Pack<R, VEC * NPL> yv;                      /* the matching VEC elements of column s of Y */
               if constexpr (YWIDE) load_wide<R, VEC * NPL>(yv, reinterpret_cast<const char *>(p.Y + ((int64_t)k + (int64_t)s * p.sYs) * NPL));
               else
               {
#pragma unroll
                  for (int v = 0; v < VEC; v++)
                  {  const R *yp = p.Y + ((int64_t)(k + v) * p.sYk + (int64_t)s * p.sYs) * NPL;
                     yv.v[v * NPL] = yp[0]; if (CPLX) yv.v[v * NPL + 1] = yp[1];
                  }
               }
#pragma unroll
               for (int v = 0; v < VEC; v++)
               {  if (!CPLX) ar[s] += (double)xv.v[v] * (double)yv.v[v];
                  else
                  {  const double xr = xv.v[2 * v], xi = p.conjX ? -(double)xv.v[2 * v + 1] : (double)xv.v[2 * v + 1];
                     const double yr = yv.v[2 * v], yi = p.conjY ? -(double)yv.v[2 * v + 1] : (double)yv.v[2 * v + 1];
                     ar[s] += xr * yr - xi * yi; ai[s] += xr * yi + xi * yr;
                  }
               }
            }
         }
      };
      const uint32_t step = G * VEC;
      uint32_t k = lane * VEC;
      for (; k + 3 * step < kfull; k += 4 * step)         /* four loads of the large operand in flight */
      {  Pack<R, VEC * NPL> xv[4];
#pragma unroll
         for (int u = 0; u < 4; u++) fetch(xv[u], k + u * step);
#pragma unroll
         for (int u = 0; u < 4; u++) accumulate(xv[u], k + u * step);
      }
      for (; k < kfull; k += step) { Pack<R, VEC * NPL> xv; fetch(xv, k); accumulate(xv, k); }
      if (lane == 0)                                    /* the K % VEC last elements */
         for (uint32_t k = kfull; k < p.K; k++)
#pragma unroll
            for (int s = 0; s < S; s++)
            {  if (s < (int)p.S)
               {  const R *xp = x + (int64_t)k * NPL, *yp = p.Y + ((int64_t)k * p.sYk + (int64_t)s * p.sYs) * NPL;
                  if (!CPLX) ar[s] += (double)xp[0] * (double)yp[0];
                  else
                  {  const double xr = xp[0], xi = p.conjX ? -(double)xp[1] : (double)xp[1];
                     const double yr = yp[0], yi = p.conjY ? -(double)yp[1] : (double)yp[1];
                     ar[s] += xr * yr - xi * yi; ai[s] += xr * yi + xi * yr;
                  }
               }
            }
   }
#pragma unroll
   for (int s = 0; s < S; s++)
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1)
         if ((uint32_t)m < G) { ar[s] += __shfl_xor(ar[s], m, 64); if (CPLX) ai[s] += __shfl_xor(ai[s], m, 64); }
   if (active && lane == 0)
   {  double alr, ali, ber, bei;
      gemv_scalars<R, CPLX>(p, alr, ali, ber, bei);
#pragma unroll
      for (int s = 0; s < S; s++) if (s < (int)p.S) gemv_store<R, CPLX>(p, row, s, ar[s], CPLX ? ai[s] : 0.0, alr, ali, ber, bei);
   }
}

/* host side: returns 1 when the product was launched here, 0 when the caller should use the tiled kernels, -1 on error */
template <class R, bool CPLX>
static int launch_gemv(const GemvParams<R> &in, hipStream_t stream)
{
   constexpr int NPL = CPLX ? 2 : 1;
   constexpr int ES = (int)sizeof(R) * NPL;
   constexpr int VEC = (16 / ES) > 0 ? 16 / ES : 1;
   GemvParams<R> p = in;
   auto aligned16 = [](const void *q) { return ((uintptr_t)q % 16) == 0; };
#define OCH_GEMV_BY_S(KERNEL, V, GRID)                                                                            \
   do { if (p.S == 1)      hipLaunchKernelGGL((KERNEL<R, CPLX, 1, V>), GRID, dim3(256), 0, stream, p);            \
        else if (p.S <= 4) hipLaunchKernelGGL((KERNEL<R, CPLX, 4, V>), GRID, dim3(256), 0, stream, p);            \
        else               hipLaunchKernelGGL((KERNEL<R, CPLX, 8, V>), GRID, dim3(256), 0, stream, p); } while (0)
   if (p.sXr == 1)
   {  const bool wide = VEC > 1 && p.rows % VEC == 0 && aligned16(p.X) && ((p.sXk * ES) % 16 == 0);
      const uint32_t per_block = 256 * (wide ? VEC : 1);
      const uint32_t rowblocks = (p.rows + per_block - 1) / per_block;
      /* enough blocks to fill the device; a slice is at least 32 long; the partial results must fit the workspace */
      uint64_t slices = (1024 + rowblocks - 1) / rowblocks;
      if (slices > 64) slices = 64;
      if (slices > p.K / 32) slices = p.K / 32;
      const uint64_t fit = OCH_GEMM_WORKSPACE / ((uint64_t)p.rows * p.S * NPL * sizeof(double));
      if (slices > fit) slices = fit;
      if (slices > 65535) slices = 65535;
      if (slices < 1) slices = 1;
      p.kper = (uint32_t)((p.K + slices - 1) / slices);
      p.slices = (p.kper > 0) ? (p.K + p.kper - 1) / p.kper : 1;
      if (p.slices < 1) p.slices = 1;
      if (p.slices > 1)
      {  char *ws;
         if (stream_gemm_workspace(stream, &ws) != 0) return -1;
         p.partials = reinterpret_cast<double *>(ws);
      }
      const dim3 grid(rowblocks, p.slices);
      if (wide) OCH_GEMV_BY_S(gemv_rows_kernel, VEC, grid); else OCH_GEMV_BY_S(gemv_rows_kernel, 1, grid);
      if (p.slices > 1)
         hipLaunchKernelGGL((gemv_finish_kernel<R, CPLX>), dim3((unsigned)(((uint64_t)p.rows * p.S + 255) / 256)), dim3(256), 0, stream, p);
   }
   else if (p.sXk == 1)
   {  const bool wide = VEC > 1 && aligned16(p.X) && ((p.sXr * ES) % 16 == 0);
      const uint32_t loads = p.K / (wide ? VEC : 1);
      p.lanes = 64;
      while (p.lanes > 8 && (p.lanes / 2) * 4 >= loads) p.lanes /= 2;
      const uint32_t per_block = 256 / p.lanes;
      const dim3 grid((p.rows + per_block - 1) / per_block);
      const bool ywide = wide && p.sYk == 1 && aligned16(p.Y) && (p.S == 1 || (p.sYs * ES) % 16 == 0);
      if (ywide)
      {  if (p.S == 1)      hipLaunchKernelGGL((gemv_dots_kernel<R, CPLX, 1, VEC, true>), grid, dim3(256), 0, stream, p);
         else if (p.S <= 4) hipLaunchKernelGGL((gemv_dots_kernel<R, CPLX, 4, VEC, true>), grid, dim3(256), 0, stream, p);
         else               hipLaunchKernelGGL((gemv_dots_kernel<R, CPLX, 8, VEC, true>), grid, dim3(256), 0, stream, p);
      }
      else if (wide) OCH_GEMV_BY_S(gemv_dots_kernel, VEC, grid); else OCH_GEMV_BY_S(gemv_dots_kernel, 1, grid);
   }
   else return 0;
#undef OCH_GEMV_BY_S
   if (hipGetLastError() != hipSuccess) { set_error("kernel launch failed (matrix-vector product)"); return -1; }
   return 1;
}

} /* namespace och */
