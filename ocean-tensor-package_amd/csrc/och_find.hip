/* Find / mask-to-offset on the device: stream compaction of the non-zero positions of a bool tensor.
 * Replaces the CPU-only solid_cpu_find_prepare / find_apply (solid/src/core/cpu/template_index.c:296-500).
 *
 *   count : every block counts the non-zero elements of one chunk of OCH_FIND_CHUNK consecutive elements
 *           (dimension 0 fastest) into workspace[1 + chunk]
 *   scan  : one block turns the counts into start positions in place (exclusive prefix sum), the total goes to
 *           workspace[0], which the host reads back
 *   apply : every block recomputes its chunk, ranks its non-zero elements with a block-wide prefix sum
 *           (wave scan + LDS), compacts their positions in LDS and writes indices or offsets from start[chunk] on
 * A thread looks at 16 consecutive elements; where these are 16 aligned consecutive bytes it takes them in one load.
 * The output order is deterministic: the order of the elements themselves.
 */
#include "och_elemwise.h"

namespace och {

#define OCH_FIND_THREADS 256
#define OCH_FIND_PER_THREAD 16
#define OCH_FIND_CHUNK (OCH_FIND_THREADS * OCH_FIND_PER_THREAD)

struct FindParams
{
   const char *ptr;
   uint64_t    nelem;
   int         ndims;
   FastDiv     div[OCH_MAX_DIMS];
   int64_t     strides[OCH_MAX_DIMS];
   int64_t     mult[OCH_MAX_DIMS];
   int         offsets;             /* 1: write sum of index * mult; 0: write the indices */
   int         wide;                /* 1: every aligned run of 16 elements is 16 consecutive, 16-byte aligned bytes */
};

/* flat element number -> indices (dimension 0 fastest); returns the byte offset. Element counts below 2^32 use the
   multiply-shift division, larger ones 64-bit division */
OCH_D int64_t find_decompose(const FindParams &p, uint64_t e, uint32_t (&idx)[OCH_MAX_DIMS])
{  int64_t off = 0;
   if (p.nelem <= 0xFFFFFFFFull)
   {  uint32_t q = (uint32_t)e;
      for (int d = 0; d < p.ndims; d++)
      {  uint32_t q2 = fastdiv(q, p.div[d]);
         idx[d] = q - q2 * p.div[d].d; q = q2; off += (int64_t)idx[d] * p.strides[d];
      }
   }
   else
   {  uint64_t q = e;
      for (int d = 0; d < p.ndims; d++)
      {  uint64_t q2 = q / p.div[d].d;
         idx[d] = (uint32_t)(q - q2 * p.div[d].d); q = q2; off += (int64_t)idx[d] * p.strides[d];
      }
   }
   return off;
}
/* advance indices and offset to the next element; past the last element the result is not used */
OCH_D void find_step(const FindParams &p, uint32_t (&idx)[OCH_MAX_DIMS], int64_t &off)
{  for (int d = 0; d < p.ndims; d++)
   {  idx[d]++; off += p.strides[d];
      if (idx[d] < p.div[d].d || d + 1 == p.ndims) return;
      off -= (int64_t)p.div[d].d * p.strides[d]; idx[d] = 0;
   }
}
/* four bytes -> four bits: bit k set iff byte k is non-zero */
OCH_D unsigned int find_nibble(uint32_t w)
{  const uint32_t t = ((((w & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | w) & 0x80808080u) >> 7;   /* bits 0, 8, 16, 24 */
   return (t * 0x01020408u) >> 24;                /* the four products that land in bits 24..27 do not collide */
}
/* bit k of the result: element base + k exists and is non-zero */
OCH_D unsigned int find_flags(const FindParams &p, uint64_t base)
{  unsigned int flags = 0; uint32_t idx[OCH_MAX_DIMS];
   if (base >= p.nelem) return 0;
   int64_t off = find_decompose(p, base, idx);
   if (p.wide)
   {  const uint4 w = *(const uint4 *)(p.ptr + off);
      return find_nibble(w.x) | (find_nibble(w.y) << 4) | (find_nibble(w.z) << 8) | (find_nibble(w.w) << 12);
   }
   for (int k = 0; k < OCH_FIND_PER_THREAD && base + k < p.nelem; k++)
   {  if (p.ptr[off] != 0) flags |= 1u << k;
      find_step(p, idx, off);
   }
   return flags;
}

__global__ __launch_bounds__(OCH_FIND_THREADS) void find_count_kernel(const FindParams p, unsigned long long *workspace)
{
   __shared__ unsigned int lds[OCH_FIND_THREADS / 64];
   const uint64_t base = (uint64_t)blockIdx.x * OCH_FIND_CHUNK + (uint64_t)threadIdx.x * OCH_FIND_PER_THREAD;
   unsigned int c = __popc(find_flags(p, base));
   for (int m = 32; m >= 1; m >>= 1) c += __shfl_xor(c, m, 64);
   if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = c;
   __syncthreads();
   if (threadIdx.x == 0) workspace[1 + blockIdx.x] = (unsigned long long)lds[0] + lds[1] + lds[2] + lds[3];
}

/* exclusive prefix sum of workspace[1 .. 1 + n) in place; total to workspace[0] */
__global__ __launch_bounds__(1024) void find_scan_kernel(unsigned long long *workspace, uint64_t n)
{
   __shared__ unsigned long long part[1024];
   const uint64_t per = (n + 1023) / 1024, lo = (uint64_t)threadIdx.x * per, hi = (lo + per < n) ? lo + per : n;
   unsigned long long s = 0;
   for (uint64_t i = lo; i < hi; i++) s += workspace[1 + i];
   part[threadIdx.x] = s;
   __syncthreads();
   if (threadIdx.x == 0)
   {  unsigned long long run = 0;
      for (int t = 0; t < 1024; t++) { unsigned long long v = part[t]; part[t] = run; run += v; }
      workspace[0] = run;
   }
   __syncthreads();
   unsigned long long run = part[threadIdx.x];
   for (uint64_t i = lo; i < hi; i++) { unsigned long long v = workspace[1 + i]; workspace[1 + i] = run; run += v; }
}

/* The non-zero elements of the chunk are first compacted in LDS (their position within the chunk, in element order);
   the threads then write the results side by side, so that the stores of a wave cover consecutive output entries. */
__global__ __launch_bounds__(OCH_FIND_THREADS) void find_apply_kernel(const FindParams p, const unsigned long long *workspace, int64_t *out)
{
   __shared__ unsigned int lds[OCH_FIND_THREADS / 64];
   __shared__ unsigned short where[OCH_FIND_CHUNK];
   const uint64_t chunk = (uint64_t)blockIdx.x * OCH_FIND_CHUNK;
   const unsigned int flags = find_flags(p, chunk + (uint64_t)threadIdx.x * OCH_FIND_PER_THREAD), c = __popc(flags);
   unsigned int incl = c;
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   for (int d = 1; d < 64; d <<= 1) { unsigned int v = __shfl_up(incl, d, 64); if (lane >= d) incl += v; }
   if (lane == 63) lds[wave] = incl;
   __syncthreads();
   unsigned int before = 0, total = 0;
   for (int w = 0; w < OCH_FIND_THREADS / 64; w++) { if (w < wave) before += lds[w]; total += lds[w]; }
   unsigned int rank = before + (incl - c);
   for (unsigned int f = flags; f; f &= f - 1)
      where[rank++] = (unsigned short)(threadIdx.x * OCH_FIND_PER_THREAD + (__ffs(f) - 1));
   __syncthreads();
   const uint64_t start = workspace[1 + blockIdx.x];
   for (unsigned int j = threadIdx.x; j < total; j += OCH_FIND_THREADS)
   {  const uint64_t e = chunk + where[j];
      if (p.ndims == 1) { out[start + j] = p.offsets ? (int64_t)e * p.mult[0] : (int64_t)e; continue; }
      uint32_t idx[OCH_MAX_DIMS];
      find_decompose(p, e, idx);
      if (p.offsets)
      {  int64_t s = 0;
         for (int d = 0; d < p.ndims; d++) s += (int64_t)idx[d] * p.mult[d];
         out[start + j] = s;
      }
      else for (int d = 0; d < p.ndims; d++) out[(start + j) * p.ndims + d] = idx[d];
   }
}

static int find_params(FindParams &p, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr)
{
   if (ndims < 0 || ndims > OCH_MAX_DIMS) return set_error("invalid number of dimensions (%d)", ndims);
   memset(&p, 0, sizeof(p));
   p.ptr = (const char *)ptr; p.ndims = ndims; p.nelem = 1;
   for (int d = 0; d < ndims; d++)
   {  if (size[d] > 0xFFFFFFFFull) return set_error("find: dimension %d is too large", d);
      if (size[d] && p.nelem > 0x7FFFFFFFFFFFull / size[d]) return set_error("find: too many elements");
      p.nelem *= size[d]; p.div[d] = make_fastdiv((uint32_t)(size[d] ? size[d] : 1)); p.strides[d] = strides[d];
   }
   if (p.nelem > 0 && ptr == nullptr) return set_error("find: null data pointer");
   /* runs of 16 elements are 16 aligned bytes when dimension 0 is dense, a multiple of 16 long, and every row starts aligned */
   p.wide = (ndims >= 1 && p.nelem > 0 && strides[0] == 1 && size[0] % 16 == 0 && ((uintptr_t)ptr & 15) == 0);
   for (int d = 1; d < ndims && p.wide; d++) if (size[d] > 1 && (strides[d] & 15) != 0) p.wide = 0;
   return 0;
}

} /* namespace och */

using namespace och;

extern "C" size_t och_find_workspace_size(size_t nelem)
{  return (2 + (nelem + OCH_FIND_CHUNK - 1) / OCH_FIND_CHUNK) * sizeof(unsigned long long); }

extern "C" int och_find_count(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, void *workspace, size_t *nnz, och_stream stream)
{
   FindParams p; unsigned long long total = 0;
   if (!workspace || !nnz) return set_error("find: null argument");
   if (find_params(p, ndims, size, strides, ptr) != 0) return -1;
   *nnz = 0;
   if (p.nelem == 0) return fill_bytes(workspace, 0, 2 * sizeof(unsigned long long), as_stream(stream));
   const uint64_t chunks = (p.nelem + OCH_FIND_CHUNK - 1) / OCH_FIND_CHUNK;
   if (chunks > 0x7FFFFFFFull) return set_error("find: too many elements");
   hipLaunchKernelGGL(find_count_kernel, dim3((unsigned)chunks), dim3(OCH_FIND_THREADS), 0, as_stream(stream), p, (unsigned long long *)workspace);
   hipLaunchKernelGGL(find_scan_kernel, dim3(1), dim3(1024), 0, as_stream(stream), (unsigned long long *)workspace, chunks);
   OCH_CHECK_LAUNCH();
   OCH_CHECK_HIP(hipMemcpyAsync(&total, workspace, sizeof(total), hipMemcpyDeviceToHost, as_stream(stream)));
   OCH_CHECK_HIP(hipStreamSynchronize(as_stream(stream)));
   *nnz = (size_t)total;
   return 0;
}

extern "C" int och_find_apply(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, void *workspace,
                              const int64_t *multiplier, int64_t *out, och_stream stream)
{
   FindParams p;
   if (!workspace) return set_error("find: null argument");
   if (find_params(p, ndims, size, strides, ptr) != 0) return -1;
   if (p.nelem == 0) return 0;
   if (multiplier) { p.offsets = 1; for (int d = 0; d < ndims; d++) p.mult[d] = multiplier[d]; }
   const uint64_t chunks = (p.nelem + OCH_FIND_CHUNK - 1) / OCH_FIND_CHUNK;
   hipLaunchKernelGGL(find_apply_kernel, dim3((unsigned)chunks), dim3(OCH_FIND_THREADS), 0, as_stream(stream), p, (const unsigned long long *)workspace, out);
   OCH_CHECK_LAUNCH();
   return 0;
}
