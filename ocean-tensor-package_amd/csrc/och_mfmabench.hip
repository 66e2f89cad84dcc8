/* Matrix-core micro-benchmark (no counterpart in the reference): what a loop of nothing but MFMAs sustains on this
 * device, and what other instructions of the same wave cost when they stand between the MFMAs. The GEMM kernels are
 * set against the first figure and are built around the second (och_gemm_f32p.hip).
 *
 * Every wave runs `iters` times through 16 MFMAs on independent accumulators, each followed by `per_mfma` instructions
 * of the kind asked for, behind a scheduling fence so that the order written is the order issued. One block of
 * 64 * waves threads per compute unit, waves = 4 or 8 (one or two waves per SIMD).
 */
#include "och_common.h"
#include "../../include/ocean_hip_bench.h"
#include <vector>
#include <algorithm>
#pragma clang diagnostic ignored "-Winline-asm"

namespace och {

typedef float    mfb_f32x16 __attribute__((ext_vector_type(16)));
typedef float    mfb_f32x4  __attribute__((ext_vector_type(4)));
typedef double   mfb_f64x4  __attribute__((ext_vector_type(4)));
typedef _Float16 mfb_h8     __attribute__((ext_vector_type(8)));
typedef int      mfb_i32x4  __attribute__((ext_vector_type(4)));
typedef int      mfb_i32x16 __attribute__((ext_vector_type(16)));

/* TYPE: 0 float 32x32x2, 1 double 16x16x4, 2 half 32x32x16, 3 int8 32x32x32 */
template <int TYPE> struct MfbOp;
template <> struct MfbOp<0>
{  typedef mfb_f32x16 Acc; typedef float In; static constexpr int ACCS = 8; static constexpr double FLOP = 2.0 * 32 * 32 * 2;
   static __device__ __forceinline__ In make(float x) { return x; }
   static __device__ __forceinline__ Acc mma(In a, In b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};
template <> struct MfbOp<1>
{  typedef mfb_f64x4 Acc; typedef double In; static constexpr int ACCS = 16; static constexpr double FLOP = 2.0 * 16 * 16 * 4;
   static __device__ __forceinline__ In make(float x) { return x; }
   static __device__ __forceinline__ Acc mma(In a, In b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
};
template <> struct MfbOp<2>
{  typedef mfb_f32x16 Acc; typedef mfb_h8 In; static constexpr int ACCS = 8; static constexpr double FLOP = 2.0 * 32 * 32 * 16;
   static __device__ __forceinline__ In make(float x) { In v; for (int i = 0; i < 8; i++) v[i] = (_Float16)(x * (0.5f + 0.37f * i) - 0.11f * i); return v; }
   static __device__ __forceinline__ Acc mma(In a, In b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct MfbOp<3>
{  typedef mfb_i32x16 Acc; typedef mfb_i32x4 In; static constexpr int ACCS = 8; static constexpr double FLOP = 2.0 * 32 * 32 * 32;
   static __device__ __forceinline__ In make(float x) { In v; for (int i = 0; i < 4; i++) v[i] = __float_as_int(x) * (2 * i + 3) + (__float_as_int(x) >> (3 * i + 5)); return v; }
   static __device__ __forceinline__ Acc mma(In a, In b, Acc c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
};

/* KIND: 0 nothing, 1 v_mov_b32, 2 v_add_f32, 3 s_nop, 4 s_add_u32, 5 s_waitcnt (nothing to wait for), 6 ds_read_b128,
   7 nothing, and every MFMA on the same pair of operands */
template <int TYPE, int KIND, int N, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void mfmabench_kernel(float *out, const float *in, int iters)
{
   typedef MfbOp<TYPE> Op;
   __shared__ mfb_f32x4 lds[64 * WAVES];
   typename Op::Acc acc[Op::ACCS];
#pragma unroll
   for (int i = 0; i < Op::ACCS; i++)
#pragma unroll
      for (int r = 0; r < (int)(sizeof(typename Op::Acc) / sizeof(acc[0][0])); r++) acc[i][r] = 0;
   /* double: the compiler keeps such accumulators in ordinary registers and copies them to the accumulation registers and
      back around every MFMA, so here the 16 tiles are addressed by name, a[8 t : 8 t + 7], as in och_gemm_f64p.hip */
   if (TYPE == 1) asm volatile(".set och_mfb, 0\n\t.rept 128\n\tv_accvgpr_write_b32 a[och_mfb], 0\n\t.set och_mfb, och_mfb + 1\n\t.endr" : : : "a127");
   /* four operands each way from pseudo-random input, a different pair for every MFMA of an iteration: the power the
      matrix cores draw, and with it the clock, depends on how the operand bits change from one MFMA to the next */
   const float x = in[threadIdx.x], y = in[threadIdx.x + 64];
   typename Op::In a[4], b[4];
#pragma unroll
   for (int k = 0; k < 4; k++) { a[k] = Op::make(in[threadIdx.x + 128 * k]); b[k] = Op::make(in[threadIdx.x + 128 * k + 64]); }
   lds[threadIdx.x] = mfb_f32x4{x, y, x, y};
   __syncthreads();
   float t = x; unsigned s = 0; mfb_f32x4 q = {0, 0, 0, 0};
   const unsigned ldsaddr = threadIdx.x * 16;
   for (int it = 0; it < iters; it++)
   {
#pragma unroll
      for (int c = 0; c < 16; c++)
      {  if (TYPE == 1) asm volatile("v_mfma_f64_16x16x4_f64 a[%2:%2+7], %0, %1, a[%2:%2+7]" : : "v"(a[KIND == 7 ? 0 : c % 4]), "v"(b[KIND == 7 ? 0 : c / 4]), "i"(8 * (c % 16)));
         else acc[c % Op::ACCS] = Op::mma(a[KIND == 7 ? 0 : c % 4], b[KIND == 7 ? 0 : c / 4], acc[c % Op::ACCS]);
#pragma unroll
         for (int n = 0; n < N; n++)
         {  if (KIND == 1) asm volatile("v_mov_b32 %0, %1" : "=v"(t) : "v"(x));
            if (KIND == 2) asm volatile("v_add_f32 %0, %1, %1" : "=v"(t) : "v"(x));
            if (KIND == 3) asm volatile("s_nop 0");
            if (KIND == 4) asm volatile("s_add_u32 %0, %0, 1" : "+s"(s) : : "scc");
            if (KIND == 5) asm volatile("s_waitcnt lgkmcnt(0)");
            if (KIND == 6) asm volatile("ds_read_b128 %0, %1" : "=v"(q) : "v"(ldsaddr));
         }
         __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile("s_waitcnt lgkmcnt(0)");
   }
   float r = t + (float)s + q.x;
#pragma unroll
   for (int i = 0; i < Op::ACCS; i++) r += (float)acc[i][0] + (float)acc[i][1];
   out[blockIdx.x * blockDim.x + threadIdx.x] = r;
}

typedef void (*mfb_kernel)(float *, const float *, int);
template <int TYPE, int KIND, int N> static mfb_kernel mfb_pick_waves(int waves)
{  return waves == 4 ? (mfb_kernel)mfmabench_kernel<TYPE, KIND, N, 4> : (mfb_kernel)mfmabench_kernel<TYPE, KIND, N, 8>; }
template <int TYPE, int KIND> static mfb_kernel mfb_pick_n(int n, int waves)
{  switch (n)
   {  case 0: return mfb_pick_waves<TYPE, 0, 0>(waves);
      case 1: return mfb_pick_waves<TYPE, KIND, 1>(waves);
      case 2: return mfb_pick_waves<TYPE, KIND, 2>(waves);
      case 4: return mfb_pick_waves<TYPE, KIND, 4>(waves);
   }
   return nullptr;
}
template <int TYPE> static mfb_kernel mfb_pick_kind(int kind, int n, int waves)
{  switch (kind)
   {  case 0: return mfb_pick_n<TYPE, 0>(0, waves);
      case 7: return mfb_pick_waves<TYPE, 7, 0>(waves);
      case 1: return mfb_pick_n<TYPE, 1>(n, waves); case 2: return mfb_pick_n<TYPE, 2>(n, waves); case 3: return mfb_pick_n<TYPE, 3>(n, waves);
      case 4: return mfb_pick_n<TYPE, 4>(n, waves); case 5: return mfb_pick_n<TYPE, 5>(n, waves); case 6: return mfb_pick_n<TYPE, 6>(n, waves);
   }
   return nullptr;
}

}  /* namespace och */

using namespace och;

/* type: 0 float, 1 double, 2 half, 3 int8 MFMA. kind: 0 MFMAs alone (16 pairs of pseudo-random operands in turn), 7 MFMAs
   alone on one pair of operands, 1 v_mov_b32, 2 v_add_f32, 3 s_nop, 4 s_add_u32, 5 s_waitcnt, 6 ds_read_b128 -- `per_mfma`
   (1, 2 or 4; ignored for kinds 0 and 7) of them after every MFMA. waves: 4 or 8 per
   block (one block per compute unit). Times `reps` launches of `iters` iterations of 16 MFMAs per wave with events on
   `stream` after one untimed launch; returns the median time of a launch and the flop it performs. Synchronous. */
extern "C" int och_mfmabench(int type, int kind, int per_mfma, int waves, int iters, int reps, float *median_ms, double *flop, och_stream stream_)
{
   hipStream_t stream = as_stream(stream_);
   if (type < 0 || type > 3 || kind < 0 || kind > 7) return set_error("mfmabench: unknown type %d or kind %d", type, kind);
   if (waves != 4 && waves != 8) return set_error("mfmabench: 4 or 8 waves per block");
   if (iters < 1 || iters > (1 << 20) || reps < 1 || reps > 1000) return set_error("mfmabench: iters / reps out of range");
   mfb_kernel fn = nullptr;
   switch (type)
   {  case 0: fn = mfb_pick_kind<0>(kind, per_mfma, waves); break; case 1: fn = mfb_pick_kind<1>(kind, per_mfma, waves); break;
      case 2: fn = mfb_pick_kind<2>(kind, per_mfma, waves); break; case 3: fn = mfb_pick_kind<3>(kind, per_mfma, waves); break;
   }
   if (fn == nullptr) return set_error("mfmabench: per_mfma must be 1, 2 or 4");
   const int blocks = gemm_compute_units();
   static const double flop_per_mfma[4] = { MfbOp<0>::FLOP, MfbOp<1>::FLOP, MfbOp<2>::FLOP, MfbOp<3>::FLOP };
   *flop = flop_per_mfma[type] * 16.0 * iters * waves * blocks;
   float *in = nullptr, *out = nullptr;
   OCH_CHECK_HIP(hipMalloc(&in, 4096));
   if (hipMalloc(&out, (size_t)blocks * 64 * waves * 4) != hipSuccess) { (void)hipFree(in); return set_error("mfmabench: hipMalloc failed"); }
   {  float host[1024];
      unsigned int state = 12345u;
      for (int i = 0; i < 1024; i++) { state = state * 1664525u + 1013904223u; host[i] = (float)(int)(state >> 8) / 8388608.0f - 1.0f; }
      if (hipMemcpy(in, host, sizeof(host), hipMemcpyHostToDevice) != hipSuccess) { (void)hipFree(in); (void)hipFree(out); return set_error("mfmabench: copy of the operands failed"); }
   }
   hipEvent_t e0, e1;
   if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { (void)hipFree(in); (void)hipFree(out); return set_error("mfmabench: event creation failed"); }
   std::vector<float> ms;
   int status = 0;
   for (int r = -1; r < reps && status == 0; r++)
   {  (void)hipEventRecord(e0, stream);
      hipLaunchKernelGGL(fn, dim3(blocks), dim3(64 * waves), 0, stream, out, in, iters);
      (void)hipEventRecord(e1, stream);
      float t = 0;
      if (hipGetLastError() != hipSuccess || hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&t, e0, e1) != hipSuccess)
         status = set_error("mfmabench: launch or timing failed");
      else if (r >= 0) ms.push_back(t);
   }
   (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
   (void)hipFree(in); (void)hipFree(out);
   if (status != 0) return status;
   std::sort(ms.begin(), ms.end());
   *median_ms = ms[ms.size() / 2];
   return 0;
}
