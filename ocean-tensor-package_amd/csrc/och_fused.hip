/* Fused projection step of a modified Gram-Schmidt sweep: v is made orthogonal to k columns, one after the other,
 * in one launch. The reference has no such entry; its callers spend two launches per pair of columns (a dot product
 * through gemm, src/core/gpu/op/tensor_blas_gpu.c:63-255, and a rank-1 update), and at 4096 elements per column both
 * are pure launch latency.
 *
 * One workgroup of 1024 threads keeps v in registers (element t of v lives in thread t mod 1024). Per column: every
 * thread multiplies its elements, the waves reduce with DPP moves (no LDS traffic), their partial sums meet in LDS (two
 * buffers in turn: one barrier per column), every row of 16 lanes adds them in the same tree and every thread updates
 * its part of v. Columns are loaded
 * several ahead of their use (as many as 256 bytes of registers per thread hold, at most 8), so that memory latency overlaps the
 * reductions of the columns before.
 */
#include "och_gemm.h"
#include "../../include/ocean_hip.h"

namespace och {

#define OCH_MGS_THREADS 1024
#define OCH_MGS_MAX_PER_THREAD 16

/* x of the lane that the DPP control names (within rows of 16 lanes): two 32-bit moves */
template <int CTRL> __device__ __forceinline__ double dpp_move(double x)
{  int lo = __double2loint(x), hi = __double2hiint(x);
   lo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xF, 0xF, false);
   hi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xF, 0xF, false);
   return __hiloint2double(hi, lo);
}
/* sum over every row of 16 lanes, in all of its lanes: lanes 1 and 2 apart (quad permutations), then the mirrored half
   row and the mirrored row. A fixed tree: the same result in every lane and on every run. */
__device__ __forceinline__ double row_sum(double x)
{  x += dpp_move<0xB1>(x);          /* quad_perm [1, 0, 3, 2] */
   x += dpp_move<0x4E>(x);          /* quad_perm [2, 3, 0, 1] */
   x += dpp_move<0x141>(x);         /* row_half_mirror */
   x += dpp_move<0x140>(x);         /* row_mirror */
   return x;
}
__device__ __forceinline__ double lane_value(double x, int lane)
{  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(x), lane), __builtin_amdgcn_readlane(__double2loint(x), lane)); }
/* sum over the wave, in all lanes */
__device__ __forceinline__ double wave_sum(double x)
{  x = row_sum(x);
   return (lane_value(x, 0) + lane_value(x, 16)) + (lane_value(x, 32) + lane_value(x, 48));
}

template <class R, bool CPLX> struct MgsElem { R re, im; };
template <class R> struct MgsElem<R, false> { R re; };

template <class R, bool CPLX, int PT, int D, int THREADS>
__global__ __launch_bounds__(THREADS) void mgs_project_kernel(uint32_t n, uint32_t k, const char *Q, int64_t ldq_bytes, char *v, char *r)
{
   typedef MgsElem<R, CPLX> E;
   static_assert(THREADS / 64 <= 16, "the partial sums of the waves are added by one row of 16 lanes");
   __shared__ double part[2][2][16];             /* [buffer][real, imaginary][wave], unused waves stay zero */
   if (threadIdx.x < 64) part[threadIdx.x >> 5][(threadIdx.x >> 4) & 1][threadIdx.x & 15] = 0;
   __syncthreads();
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   E x[PT], q[D][PT];                           /* q[d]: this thread's elements of column i + d, loaded D columns ahead */
   const E zero = {};
#pragma unroll
   for (int e = 0; e < PT; e++)
   {  const uint32_t t = threadIdx.x + THREADS * e;
      x[e] = (t < n) ? reinterpret_cast<const E *>(v)[t] : zero;
#pragma unroll
      for (int d = 0; d < D; d++)
         q[d][e] = (t < n && (uint32_t)d < k) ? reinterpret_cast<const E *>(Q + (int64_t)d * ldq_bytes)[t] : zero;
   }
   for (uint32_t i0 = 0; i0 < k; i0 += D)
   {
#pragma unroll
      for (int d = 0; d < D; d++)
      {  const uint32_t i = i0 + d;
         if (i >= k) break;
         /* r = q^H x */
         double sr = 0, si = 0;
#pragma unroll
         for (int e = 0; e < PT; e++)
         {  if constexpr (CPLX)
            {  sr += (double)q[d][e].re * (double)x[e].re + (double)q[d][e].im * (double)x[e].im;
               si += (double)q[d][e].re * (double)x[e].im - (double)q[d][e].im * (double)x[e].re;
            }
            else sr += (double)q[d][e].re * (double)x[e].re;
         }
         E cur[PT];
#pragma unroll
         for (int e = 0; e < PT; e++) cur[e] = q[d][e];
         if (i + D < k)
         {  const E *next = reinterpret_cast<const E *>(Q + (int64_t)(i + D) * ldq_bytes);
#pragma unroll
            for (int e = 0; e < PT; e++)
            {  const uint32_t t = threadIdx.x + THREADS * e;
               q[d][e] = (t < n) ? next[t] : zero;
            }
         }
         sr = wave_sum(sr); if (CPLX) si = wave_sum(si);
         if (lane == 0) { part[i & 1][0][wave] = sr; if (CPLX) part[i & 1][1][wave] = si; }
         __syncthreads();
         sr = row_sum(part[i & 1][0][lane & 15]); if (CPLX) si = row_sum(part[i & 1][1][lane & 15]);
         /* the coefficient is used as it is stored: rounded to the element type */
         const R cr = (R)sr, ci = (R)si;
         if (r != nullptr && threadIdx.x == 0)
         {  reinterpret_cast<R *>(r)[(size_t)i * (CPLX ? 2 : 1)] = cr;
            if (CPLX) reinterpret_cast<R *>(r)[(size_t)i * 2 + 1] = ci;
         }
#pragma unroll
         for (int e = 0; e < PT; e++)
         {  if constexpr (CPLX)
            {  const R pr = cr * cur[e].re - ci * cur[e].im, pi = cr * cur[e].im + ci * cur[e].re;
               x[e].re -= pr; x[e].im -= pi;
            }
            else x[e].re -= cr * cur[e].re;
         }
      }
   }
#pragma unroll
   for (int e = 0; e < PT; e++)
   {  const uint32_t t = threadIdx.x + THREADS * e;
      if (t < n) reinterpret_cast<E *>(v)[t] = x[e];
   }
}

template <class R, bool CPLX>
static int mgs_launch(size_t n, size_t k, const void *Q, ptrdiff_t ldq, void *v, void *r, hipStream_t stream)
{
   const int64_t ldq_bytes = (int64_t)ldq * (int64_t)sizeof(MgsElem<R, CPLX>);
   /* columns in flight: as many as 256 bytes of registers per thread hold, at most 8 */
#define OCH_MGS_GO(PT, T) hipLaunchKernelGGL((mgs_project_kernel<R, CPLX, PT, (PT * (int)sizeof(MgsElem<R, CPLX>) >= 256) ? 1 : (256 / (PT * (int)sizeof(MgsElem<R, CPLX>)) > 8 ? 8 : 256 / (PT * (int)sizeof(MgsElem<R, CPLX>))), T>), \
                                          dim3(1), dim3(T), 0, stream, (uint32_t)n, (uint32_t)k, (const char *)Q, ldq_bytes, (char *)v, (char *)r)
   const size_t per = (n + OCH_MGS_THREADS - 1) / OCH_MGS_THREADS;
   if (per <= 1) OCH_MGS_GO(1, OCH_MGS_THREADS); else if (per <= 2) OCH_MGS_GO(2, OCH_MGS_THREADS); else if (per <= 4) OCH_MGS_GO(4, OCH_MGS_THREADS);
   else if (per <= 8) OCH_MGS_GO(8, OCH_MGS_THREADS); else OCH_MGS_GO(16, OCH_MGS_THREADS);
#undef OCH_MGS_GO
   OCH_CHECK_LAUNCH();
   return 0;
}

} /* namespace och */

using namespace och;

extern "C" int och_mgs_project(int dtype, size_t n, size_t k, const void *Q, ptrdiff_t ldq, void *v, void *r, och_stream stream)
{
   if (dtype != OCH_FLOAT && dtype != OCH_DOUBLE && dtype != OCH_CFLOAT && dtype != OCH_CDOUBLE)
      return set_error("mgs_project is available for float, double, cfloat and cdouble (got %d)", dtype);
   if (n == 0 || k == 0) return 0;
   if (Q == nullptr || v == nullptr) return set_error("mgs_project: null pointer argument");
   if (ldq < (ptrdiff_t)n) return set_error("mgs_project: ldq = %td is smaller than n = %zu", ldq, n);
   if (k > 0xFFFFFFFFull) return set_error("mgs_project: too many columns");
   if (n <= (size_t)OCH_MGS_THREADS * OCH_MGS_MAX_PER_THREAD)
   {  switch (dtype)
      {  case OCH_FLOAT:   return mgs_launch<float, false>(n, k, Q, ldq, v, r, as_stream(stream));
         case OCH_DOUBLE:  return mgs_launch<double, false>(n, k, Q, ldq, v, r, as_stream(stream));
         case OCH_CFLOAT:  return mgs_launch<float, true>(n, k, Q, ldq, v, r, as_stream(stream));
         default:          return mgs_launch<double, true>(n, k, Q, ldq, v, r, as_stream(stream));
      }
   }
   /* long vectors: the two launches per column of the unfused sequence, coefficients kept in r */
   if (r == nullptr) return set_error("mgs_project: vectors of more than %d elements need the coefficient array", OCH_MGS_THREADS * OCH_MGS_MAX_PER_THREAD);
   const size_t es = (size_t)och_type_size[dtype];
   static const double one_d[2] = { 1.0, 0.0 }, zero_d[2] = { 0.0, 0.0 }, minus_d[2] = { -1.0, 0.0 };
   static const float one_f[2] = { 1.f, 0.f }, zero_f[2] = { 0.f, 0.f }, minus_f[2] = { -1.f, 0.f };
   const bool dbl = (dtype == OCH_DOUBLE || dtype == OCH_CDOUBLE);
   const void *one = dbl ? (const void *)one_d : (const void *)one_f, *zero = dbl ? (const void *)zero_d : (const void *)zero_f;
   const void *minus = dbl ? (const void *)minus_d : (const void *)minus_f;
   for (size_t i = 0; i < k; i++)
   {  const char *qi = (const char *)Q + i * (size_t)ldq * es; char *ri = (char *)r + i * es;
      /* r_i = q_i^H v, then v <- (-1) q_i r_i + v with r_i as the 1 x 1 operand B; alpha and beta are host scalars */
      if (och_gemm(dtype, 'C', 'N', 1, 1, n, one, qi, ldq, v, (ptrdiff_t)n, zero, ri, 1, 1, stream) != 0) return -1;
      if (och_gemm(dtype, 'N', 'N', n, 1, 1, minus, qi, ldq, ri, 1, one, v, (ptrdiff_t)n, 1, stream) != 0) return -1;
   }
   return 0;
}
