/* Streaming micro-benchmark: what this device's memory sustains for the traffic mixes of the
 * elementwise, copy and cast kernels, independent of the library's own kernels.
 *
 * No counterpart in the reference. It exists so that a measured rate of a library kernel can be
 * set against the best rate ANY simple kernel reaches for the same mix of reads and writes on the
 * same device, besides the nominal 8 TB/s. Mixes: read only, write only, copy (1 read : 1 write),
 * add (2 : 1), widening cast (4 bytes read : 8 written), narrowing gather (every second 2-byte
 * element read, 4 bytes written per element: the traffic of a step-2 int16 -> float32 copy).
 * Every mix is run in several forms (accesses in flight per thread, nontemporal hint or not, one
 * group per thread or a persistent grid that walks contiguous ranges, workgroup size); the
 * operands are filled with pseudo-random bits (bit activity changes what the memory system
 * sustains under the power limit) and several sets of operands are rotated between launches so
 * that nothing is served from the 256 MB last-level cache.
 */
#include "och_common.h"
#include "../../include/ocean_hip_bench.h"
#include "och_dtypes.h"
#include <algorithm>
#include <vector>

namespace och {

typedef unsigned int mb_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int mb_u32x2 __attribute__((ext_vector_type(2)));

template <bool NT, class V> OCH_D V mb_load(const V *p) { if constexpr (NT) return __builtin_nontemporal_load(p); else return *p; }
template <bool NT, class V> OCH_D void mb_store(V *p, V v) { if constexpr (NT) __builtin_nontemporal_store(v, p); else *p = v; }

struct MbArgs
{  const char *src0, *src1; char *dst; unsigned long long ngroups;      /* groups of 16 bytes of the NARROWEST operand */
   unsigned long long per_block;                                           /* persistent form: groups per block */
};

OCH_D mb_u32x4 mb_add_f64(mb_u32x4 a, mb_u32x4 b)
{  union { mb_u32x4 v; double d[2]; } x, y; x.v = a; y.v = b; x.d[0] += y.d[0]; x.d[1] += y.d[1]; return x.v; }

/* the work of UNR groups of one thread; all loads are issued before the first use.
   Group of kind 0-3: 16 bytes of every operand. Kind 4 (float -> double): 8 bytes loaded, 16 stored. Kind 5 (every second
   int16 -> float): 16 bytes loaded (eight int16, four of them asked for), 16 stored. Kind 6 (float -> double with 16-byte
   loads): 16 bytes loaded, the lanes of a wave exchange values so that each of the two 16-byte stores of a lane is part of
   one contiguous 1024-byte run of the wave. Kind 7 (kind 5 with four 2-byte loads in place of the 16-byte load). */
template <int KIND, int UNR, bool NT>
OCH_D void mb_groups(const MbArgs &a, unsigned long long g0, unsigned long long stride, unsigned long long end, unsigned int &sink)
{
   mb_u32x4 x[UNR], y[UNR];
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  const unsigned long long g = g0 + u * stride;
      if (g < end)
      {  if constexpr (KIND == 0 || KIND == 2 || KIND == 3 || KIND == 5 || KIND == 6) x[u] = mb_load<NT>(reinterpret_cast<const mb_u32x4 *>(a.src0) + g);
         if constexpr (KIND == 3) y[u] = mb_load<NT>(reinterpret_cast<const mb_u32x4 *>(a.src1) + g);
         if constexpr (KIND == 4) { mb_u32x2 t = mb_load<NT>(reinterpret_cast<const mb_u32x2 *>(a.src0) + g); x[u].x = t.x; x[u].y = t.y; }
         if constexpr (KIND == 7)
         {  const unsigned short *s = reinterpret_cast<const unsigned short *>(a.src0) + 8 * g;
            x[u].x = s[0]; x[u].y = s[2]; x[u].z = s[4]; x[u].w = s[6];
         }
      }
   }
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  const unsigned long long g = g0 + u * stride;
      if (g < end)
      {  if constexpr (KIND == 0) sink ^= x[u].x ^ x[u].y ^ x[u].z ^ x[u].w;
         if constexpr (KIND == 1) { mb_u32x4 v = { (unsigned)g, 1u, 2u, 3u }; mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + g, v); }
         if constexpr (KIND == 2) mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + g, x[u]);
         if constexpr (KIND == 3) mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + g, mb_add_f64(x[u], y[u]));
         if constexpr (KIND == 4)
         {  union { mb_u32x4 v; double d[2]; } r;
            r.d[0] = __uint_as_float(x[u].x); r.d[1] = __uint_as_float(x[u].y);
            mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + g, r.v);
         }
         if constexpr (KIND == 5)
         {  union { mb_u32x4 v; float f[4]; } r;
            r.f[0] = (short)(x[u].x & 0xFFFFu); r.f[1] = (short)(x[u].y & 0xFFFFu); r.f[2] = (short)(x[u].z & 0xFFFFu); r.f[3] = (short)(x[u].w & 0xFFFFu);
            mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + g, r.v);
         }
         if constexpr (KIND == 7)
         {  union { mb_u32x4 v; float f[4]; } r;
            r.f[0] = (short)x[u].x; r.f[1] = (short)x[u].y; r.f[2] = (short)x[u].z; r.f[3] = (short)x[u].w;
            mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + g, r.v);
         }
      }
      if constexpr (KIND == 6)
      {  /* every lane of the wave takes part in the exchange (the sizes used keep whole waves inside the range) */
         const int lane = threadIdx.x & 63, half = lane >> 1, odd = lane & 1;
         const unsigned int a0 = __shfl(x[u].x, half, 64), a1 = __shfl(x[u].y, half, 64), a2 = __shfl(x[u].z, half, 64), a3 = __shfl(x[u].w, half, 64);
         const unsigned int b0 = __shfl(x[u].x, 32 + half, 64), b1 = __shfl(x[u].y, 32 + half, 64), b2 = __shfl(x[u].z, 32 + half, 64), b3 = __shfl(x[u].w, 32 + half, 64);
         if (g < end)
         {  union { mb_u32x4 v; double d[2]; } lo, hi;
            lo.d[0] = __uint_as_float(odd ? a2 : a0); lo.d[1] = __uint_as_float(odd ? a3 : a1);
            hi.d[0] = __uint_as_float(odd ? b2 : b0); hi.d[1] = __uint_as_float(odd ? b3 : b1);
            const unsigned long long wave0 = g - lane;                                 /* first group of the wave */
            mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + 2 * wave0 + lane, lo.v);
            mb_store<NT>(reinterpret_cast<mb_u32x4 *>(a.dst) + 2 * wave0 + 64 + lane, hi.v);
         }
      }
   }
}

/* MAP 0: one trip, block b covers groups [b * BLOCK * UNR, (b + 1) * BLOCK * UNR); MAP 1: persistent grid, block b
   walks the contiguous range [b * per_block, (b + 1) * per_block) in trips of BLOCK * UNR groups */
template <int KIND, int UNR, bool NT, int MAP>
__global__ __launch_bounds__(1024) void membench_kernel(const MbArgs a, unsigned int *sinkout)
{
   unsigned int sink = 0;
   const unsigned long long stride = blockDim.x;
   if constexpr (MAP == 0)
      mb_groups<KIND, UNR, NT>(a, (unsigned long long)blockIdx.x * (stride * UNR) + threadIdx.x, stride, a.ngroups, sink);
   else
   {  unsigned long long g = (unsigned long long)blockIdx.x * a.per_block + threadIdx.x;
      unsigned long long end = (unsigned long long)blockIdx.x * a.per_block + a.per_block;
      if (end > a.ngroups) end = a.ngroups;
      for (; g < end; g += stride * UNR) mb_groups<KIND, UNR, NT>(a, g, stride, end, sink);
   }
   if constexpr (KIND == 0) { if (sink == 0x9E3779B9u && sinkout) *sinkout = sink; }      /* keeps the loads alive */
}

/* pseudo-random bits; as doubles / floats they are finite values of mixed sign and exponent near 1 */
__global__ __launch_bounds__(256) void membench_fill_kernel(mb_u32x4 *dst, unsigned long long ngroups, unsigned int seed, int kind)
{
   for (unsigned long long g = (unsigned long long)blockIdx.x * 256 + threadIdx.x; g < ngroups; g += (unsigned long long)gridDim.x * 256)
   {  unsigned int h[4];
      for (int i = 0; i < 4; i++)
      {  unsigned int v = (unsigned int)(g * 4 + i) * 2654435761u + seed; v ^= v >> 15; v *= 2246822519u; v ^= v >> 13; v *= 3266489917u; v ^= v >> 16; h[i] = v; }
      if (kind == 8)        /* doubles in (-2, 2): random sign and mantissa, exponent 0x3FE / 0x3FF */
      {  h[1] = (h[1] & 0x801FFFFFu) | 0x3FE00000u; h[3] = (h[3] & 0x801FFFFFu) | 0x3FE00000u; }
      else if (kind == 4)   /* floats in (-2, 2) */
         for (int i = 0; i < 4; i++) h[i] = (h[i] & 0x80FFFFFFu) | 0x3F000000u;
      mb_u32x4 v = { h[0], h[1], h[2], h[3] };
      dst[g] = v;
   }
}

typedef void (*mb_kernel)(const MbArgs, unsigned int *);
template <int KIND, int UNR, bool NT, int MAP> static mb_kernel mb_pick() { return &membench_kernel<KIND, UNR, NT, MAP>; }
template <int KIND, int UNR> static mb_kernel mb_pick2(int nt, int map)
{  if (nt) return map ? mb_pick<KIND, UNR, true, 1>() : mb_pick<KIND, UNR, true, 0>();
   return map ? mb_pick<KIND, UNR, false, 1>() : mb_pick<KIND, UNR, false, 0>();
}
template <int KIND> static mb_kernel mb_pick3(int unr, int nt, int map)
{  switch (unr) { case 1: return mb_pick2<KIND, 1>(nt, map); case 2: return mb_pick2<KIND, 2>(nt, map); case 4: return mb_pick2<KIND, 4>(nt, map); }
   return nullptr;
}

}  /* namespace och */

using namespace och;

/* kind: 0 read, 1 write, 2 copy, 3 add of doubles, 4 float -> double, 5 every second int16 -> float, 6 and 7: other
   forms of 4 and 5 (see mb_groups).
   nbytes: bytes of the NARROWEST operand of one launch (a multiple of 16); the other operands follow from the kind.
   unr in {1,2,4}; nt 0/1; map 0 (one trip per thread) or 1 (persistent, `blocks` blocks); block: threads per block.
   Allocates `nsets` sets of operands, fills them with pseudo-random bits, runs `reps` timed samples of ten back-to-back
   launches (each sample between two events on `stream`; one untimed sample first), frees everything. Returns the median and the best time of one launch and the
   bytes one launch moves (reads + writes, every byte of every operand once). */
extern "C" int och_membench(int kind, int unr, int nt, int map, int block, int blocks, size_t nbytes, int nsets, int reps,
                            float *median_ms, float *best_ms, size_t *bytes_moved, och_stream stream_)
{
   hipStream_t stream = as_stream(stream_);
   if (kind < 0 || kind > 7) return set_error("membench: unknown kind %d", kind);
   if (nbytes == 0 || nbytes % 16 != 0) return set_error("membench: the size must be a positive multiple of 16 bytes");
   if (block < 64 || block > 1024 || block % 64 != 0) return set_error("membench: block size %d", block);
   if (nsets < 1 || nsets > 16 || reps < 1 || reps > 10000) return set_error("membench: nsets / reps out of range");
   mb_kernel fn = nullptr;
   switch (kind)
   {  case 0: fn = mb_pick3<0>(unr, nt, map); break; case 1: fn = mb_pick3<1>(unr, nt, map); break;
      case 2: fn = mb_pick3<2>(unr, nt, map); break; case 3: fn = mb_pick3<3>(unr, nt, map); break;
      case 4: fn = mb_pick3<4>(unr, nt, map); break; case 5: fn = mb_pick3<5>(unr, nt, map); break;
      case 6: fn = mb_pick3<6>(unr, nt, map); break; case 7: fn = mb_pick3<7>(unr, nt, map); break;
   }
   if (fn == nullptr) return set_error("membench: unr must be 1, 2 or 4");
   /* operand sizes in bytes relative to nbytes (src0, src1, dst) and bytes of the narrowest operand per group */
   static const int mul[8][3] = { { 1, 0, 0 }, { 0, 0, 1 }, { 1, 0, 1 }, { 1, 1, 1 }, { 1, 0, 2 }, { 2, 0, 2 }, { 1, 0, 2 }, { 2, 0, 2 } };
   static const int per_group[8] = { 16, 16, 16, 16, 8, 8, 16, 8 };
   if (nbytes % (size_t)(per_group[kind] * 64) != 0) return set_error("membench: the size must be a multiple of %d bytes", per_group[kind] * 64);
   const size_t ngroups = nbytes / per_group[kind];
   const size_t sz[3] = { nbytes * mul[kind][0], nbytes * mul[kind][1], nbytes * mul[kind][2] };
   /* algorithmic bytes: of the step-2 source only every second element is asked for (nbytes of it) */
   *bytes_moved = (kind == 5 || kind == 7) ? nbytes + sz[2] : sz[0] + sz[1] + sz[2];
   std::vector<void *> bufs;
   auto release = [&]() { for (void *b : bufs) (void)hipFree(b); };
   std::vector<MbArgs> sets((size_t)nsets);
   for (int s = 0; s < nsets; s++)
   {  void *p[3] = { nullptr, nullptr, nullptr };
      for (int k = 0; k < 3; k++)
      {  if (sz[k] == 0) continue;
         hipError_t e = hipMalloc(&p[k], sz[k]);
         if (e != hipSuccess) { release(); return set_error("membench: hipMalloc of %zu bytes failed: %s", sz[k], hipGetErrorString(e)); }
         bufs.push_back(p[k]);
         const int fillkind = (kind == 3) ? 8 : ((kind == 4 || kind == 6) ? 4 : 0);
         hipLaunchKernelGGL(membench_fill_kernel, dim3(4096), dim3(256), 0, stream, (mb_u32x4 *)p[k], (unsigned long long)(sz[k] / 16), 977u * (s * 3 + k) + 1u, fillkind);
      }
      sets[s].src0 = (const char *)p[0]; sets[s].src1 = (const char *)p[1]; sets[s].dst = (char *)p[2];
      sets[s].ngroups = ngroups;
      sets[s].per_block = 0;
   }
   unsigned int grid;
   if (map == 0) grid = (unsigned int)((ngroups + (size_t)block * unr - 1) / ((size_t)block * unr));
   else
   {  if (blocks < 1) blocks = 512;
      const size_t step = (size_t)block * unr;
      size_t per = (ngroups + blocks - 1) / blocks; per = (per + step - 1) / step * step;
      for (auto &s : sets) s.per_block = per;
      grid = (unsigned int)((ngroups + per - 1) / per);
   }
   hipEvent_t e0, e1;
   if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { release(); return set_error("membench: event creation failed"); }
   std::vector<float> ms;
   int status = 0;
   const int INNER = 10;             /* launches per timed sample, back to back: the events' own cost is spread over them */
   size_t turn = 0;
   for (int r = -1; r < reps && status == 0; r++)
   {  (void)hipEventRecord(e0, stream);
      for (int i = 0; i < INNER; i++)
         hipLaunchKernelGGL(fn, dim3(grid), dim3(block), 0, stream, sets[turn++ % (size_t)nsets], (unsigned int *)nullptr);
      (void)hipEventRecord(e1, stream);
      hipError_t e = hipEventSynchronize(e1);
      float t = 0;
      if (e == hipSuccess) e = hipEventElapsedTime(&t, e0, e1);
      if (e != hipSuccess) status = set_error("membench: %s", hipGetErrorString(e));
      else if (r >= 0) ms.push_back(t / INNER);
   }
   (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
   (void)hipStreamSynchronize(stream);
   release();
   if (status != 0) return status;
   std::sort(ms.begin(), ms.end());
   *best_ms = ms.front(); *median_ms = ms[ms.size() / 2];
   return 0;
}
