/* Single-launch full reduction for gfx950.
 *
 * Replaces the reference's accumulate + finalize kernel pair followed by a blocking copy
 * (solid/include/solid/core/gpu/reduce_all.h:136-274,365-414). One kernel:
 *   every block streams one contiguous range with <=128-bit loads, four independent loads in
 *   flight per thread -> 64-lane butterfly (shuffle) inside each wave -> LDS combine of the
 *   block's waves -> one partial per block in a scratch buffer -> the block that takes the last
 *   ticket (atomic counter) folds all partials in index order and writes the result.
 * The fold order depends only on the launch geometry, so results are reproducible run to run.
 * The result pointer may be device memory or device-visible pinned host memory.
 *
 * Cross-block hand-over: partials are written and read with relaxed agent-scope atomics (they
 * bypass the per-XCD L2, which is not coherent between XCDs), the writer waits for its stores
 * to complete and then takes its ticket with a relaxed agent-scope atomic add. A full
 * agent-scope fence per block (L2 write-back + invalidate) serialises at ~30 ns per block and
 * was measured to halve the streaming rate; the ticket itself costs ~5 ns per block, which is
 * why the grid is capped at two blocks per compute unit.
 */
#pragma once
#include "och_elemwise.h"
#include "och_reduce_ops.h"
#include <string.h>

namespace och {

#define OCH_RED_BLOCK 256
#define OCH_RED_UNR 4
#define OCH_RED_BLOCK_STREAM 512             /* threads of the workgroups that stream a large contiguous source */

template <class A> OCH_D A shfl_xor_any(A v, int mask)
{
   constexpr int NW = (sizeof(A) + 3) / 4;
   union { A a; int w[NW]; } u;
   for (int i = 0; i < NW; i++) u.w[i] = 0;
   u.a = v;
#pragma unroll
   for (int i = 0; i < NW; i++) u.w[i] = __shfl_xor(u.w[i], mask, 64);
   return u.a;
}

/* read / write an accumulator shared between workgroups: word-wise relaxed agent-scope atomics */
template <class A> OCH_D A load_shared_global(const char *addr)
{
   constexpr int NW = (sizeof(A) + 3) / 4;
   union { A a; unsigned int w[NW]; } u;
#pragma unroll
   for (int i = 0; i < NW; i++)
      u.w[i] = __hip_atomic_load(reinterpret_cast<const unsigned int *>(addr) + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
   return u.a;
}
template <class A> OCH_D void store_shared_global(char *addr, const A &a)
{
   constexpr int NW = (sizeof(A) + 3) / 4;
   union { A a; unsigned int w[NW]; } u;
#pragma unroll
   for (int i = 0; i < NW; i++) u.w[i] = 0;
   u.a = a;
#pragma unroll
   for (int i = 0; i < NW; i++)
      __hip_atomic_store(reinterpret_cast<unsigned int *>(addr) + i, u.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* reduce across the 256 threads of a block; the result is valid in thread 0 */
template <class RD, int BLOCK = OCH_RED_BLOCK> OCH_D typename RD::Acc block_reduce(typename RD::Acc a, typename RD::Acc *lds)
{
   typedef typename RD::Acc Acc;
#pragma unroll
   for (int m = 32; m >= 1; m >>= 1) a = RD::combine(a, shfl_xor_any<Acc>(a, m));
   const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
   if (lane == 0) lds[wave] = a;
   __syncthreads();
   if (threadIdx.x == 0)
   {
#pragma unroll
      for (int w = 1; w < BLOCK / 64; w++) a = RD::combine(a, lds[w]);
   }
   return a;
}

struct RedParams
{
   EwParams<1> ew;             /* source layout; ew.ngroups unused when flat */
   uint64_t ngroups;           /* total groups (VEC elements each) */
   uint64_t per_block;         /* groups per block: block b reduces the contiguous range starting at b * per_block */
   char *partials;             /* OCH_RED_MAX_BLOCKS slots */
   unsigned int *counter;      /* ticket counter, zero on entry, zero again on exit */
   void *result;
   char *tail;                 /* flat layout only: elements left over after the last full group */
   int   ntail;
   int64_t rowbytes;           /* row mode: bytes of one row of the first dimension */
   unsigned int slot_base;     /* partial slot of block 0 of this launch */
   unsigned int total_blocks;  /* blocks of all launches that share the counter: the block that draws the last ticket folds */
};

/* Number of elements one launch of a layout with several dimensions indexes (its group index is 32 bits wide). Larger
   tensors are cut along their outer dimensions into parts that are launched one after the other on the same stream:
   every part writes its blocks' partial results into its own range of slots and the block that draws the last ticket
   of the last part folds them all. och_reduce_set_part_limit lowers the number so that small tensors exercise this. */
#define OCH_RED_PART_LIMIT 0xFFFF0000ull
#define OCH_RED_MAX_PARTS 512
uint64_t reduce_part_limit();

/* Cuts `size` (ndims > 1, product above `limit`) into boxes of at most `limit` elements: whole runs of the outermost
   dimension where one index of it fits, otherwise index by index with the next dimension cut in turn. Calls
   visit(start, count) with the first index and the extent of every box in every dimension; returns the number of boxes,
   or -1 when the first dimension alone exceeds the limit (it is never cut: rows stay whole). */
template <class Visit>
static int64_t reduce_cut_parts(int ndims, const uint64_t *size, uint64_t limit, Visit visit)
{
   uint64_t start[OCH_MAX_DIMS] = { 0 }, count[OCH_MAX_DIMS], inner[OCH_MAX_DIMS + 1];
   inner[0] = 1;
   for (int d = 0; d < ndims; d++) { inner[d + 1] = inner[d] * size[d]; count[d] = size[d]; }   /* inner[d]: elements below dimension d */
   if (ndims < 1 || size[0] > limit) return -1;
   int top = ndims - 1;
   while (top > 0 && inner[top] > limit) top--;         /* dimensions above `top` are walked index by index */
   /* dimension `top` is cut into runs of `run` indices (inner[top] <= limit, so run >= 1); top == 0 keeps whole rows */
   const uint64_t run = (top == 0) ? size[0] : limit / inner[top];
   int64_t boxes = 0;
   for (int d = top + 1; d < ndims; d++) { count[d] = 1; start[d] = 0; }
   for (;;)
   {  for (uint64_t at = 0; at < size[top]; at += run)
      {  start[top] = at; count[top] = (size[top] - at < run) ? size[top] - at : run;
         visit(start, count); boxes++;
      }
      int d = top + 1;
      for (; d < ndims; d++) { if (++start[d] < size[d]) break; start[d] = 0; }
      if (d >= ndims) break;
   }
   return boxes;
}

/* Row mode: the first dimension is contiguous but its rows are not whole aligned 16-byte groups (a width that is not a
   multiple of VEC, a pitch or a start that is not a multiple of 16 bytes: sub-matrices of 1- and 2-byte types mostly).
   Group g is chunk i of row r: the ALIGNED 16 bytes at (row start rounded down to 16) + 16 i. The first and the last
   chunk of a row hold elements in front of / behind the row; [lo, hi) are the elements of the pack that belong to it.
   A chunk is loaded only when it holds at least one element of the row, so every load stays inside a 16-byte unit that
   the tensor owns part of. One load instruction per 16 bytes instead of one per element: 1000-byte rows of int8 at a
   pitch of 1024 are summed at 0.67 TB/s element by element. */
template <class T, int VEC>
OCH_D void rows_load(const RedParams &p, uint32_t g, Pack<T, VEC> &v, int &lo, int &hi)
{
   const uint32_t r = fastdiv(g, p.ew.div[0]), i = g - r * p.ew.div[0].d;
   int64_t rowoff = 0;
   uint32_t q = r;
   for (int d = 1; d < p.ew.ndims - 1; d++)
   {  const uint32_t q2 = fastdiv(q, p.ew.div[d]);
      rowoff += (int64_t)(q - q2 * p.ew.div[d].d) * p.ew.stride[0][d]; q = q2;
   }
   if (p.ew.ndims > 1) rowoff += (int64_t)q * p.ew.stride[0][p.ew.ndims - 1];
   const char *row = p.ew.ptr[0] + rowoff;
   const int64_t first = (int64_t)i * 16 - (int64_t)((uintptr_t)row & 15);       /* byte position of the chunk within the row */
   const int64_t left = p.rowbytes - first;                                       /* bytes of the row from the chunk's start on */
   lo = (first < 0) ? (int)((-first) / (int64_t)sizeof(T)) : 0;
   hi = (left <= 0) ? 0 : ((left >= 16) ? VEC : (int)(left / (int64_t)sizeof(T)));
   if (hi > lo) load_wide<T, VEC>(v, row + first);
}

/* MODE 1 (wide): the first dimension is contiguous, divisible by VEC and aligned: VEC-wide loads (compile-time, so that
   the loads stay single 128-bit instructions); MODE 2: row mode (see rows_load); MODE 0: VEC is 1 and any layout is accepted. */
template <class RD, class T, int VEC, int MODE, bool NT = false, int BLOCK = OCH_RED_BLOCK, int UNR = OCH_RED_UNR>
__global__ __launch_bounds__(BLOCK) void reduce_all_kernel(const RedParams p, const typename RD::Param prm)
{
   typedef typename RD::Acc Acc;
   __shared__ Acc lds[BLOCK / 64];
   __shared__ unsigned int ticket;
   Acc part[UNR];
#pragma unroll
   for (int u = 0; u < UNR; u++) part[u] = RD::identity();
   /* every block walks one contiguous range of groups, OCH_RED_BLOCK groups per step, so that
      the loads in flight stay close together in memory (a grid-wide stride is a large power of
      two and lands the concurrent loads on the same memory channels) */
   const uint64_t stride = BLOCK;
   uint64_t g = (uint64_t)blockIdx.x * p.per_block + threadIdx.x;
   uint64_t end = (uint64_t)blockIdx.x * p.per_block + p.per_block;
   if (end > p.ngroups) end = p.ngroups;
   const bool flat = (p.ew.ndims == 1);
   /* main loop: UNR independent groups per trip, loads first, one accumulator per group */
   for (; g + (UNR - 1) * stride < end; g += UNR * stride)
   {  Pack<T, VEC> v[UNR];
      if constexpr (MODE == 2)
      {  int lo[UNR], hi[UNR];
#pragma unroll
         for (int u = 0; u < UNR; u++) { v[u] = Pack<T, VEC>{}; rows_load<T, VEC>(p, (uint32_t)(g + u * stride), v[u], lo[u], hi[u]); }
#pragma unroll
         for (int k = 0; k < VEC; k++)
#pragma unroll
            for (int u = 0; u < UNR; u++) if (k >= lo[u] && k < hi[u]) part[u] = RD::combine(part[u], RD::load(v[u].v[k], prm));
      }
      else
      {
#pragma unroll
         for (int u = 0; u < UNR; u++)
         {  int64_t off[1];
            if (flat) off[0] = (int64_t)(g + u * stride) * p.ew.gstride[0];
            else group_offsets<1>(p.ew, (uint32_t)(g + u * stride), off);
            load_pack<T, VEC, NT>(v[u], p.ew.ptr[0] + off[0], p.ew.estride[0], MODE == 1);
         }
#pragma unroll
         for (int k = 0; k < VEC; k++)
#pragma unroll
            for (int u = 0; u < UNR; u++) part[u] = RD::combine(part[u], RD::load(v[u].v[k], prm));
      }
   }
   for (; g < end; g += stride)
   {  Pack<T, VEC> v;
      if constexpr (MODE == 2)
      {  int lo, hi;
         v = Pack<T, VEC>{};
         rows_load<T, VEC>(p, (uint32_t)g, v, lo, hi);
#pragma unroll
         for (int k = 0; k < VEC; k++) if (k >= lo && k < hi) part[0] = RD::combine(part[0], RD::load(v.v[k], prm));
      }
      else
      {  int64_t off[1];
         if (flat) off[0] = (int64_t)g * p.ew.gstride[0];
         else group_offsets<1>(p.ew, (uint32_t)g, off);
         load_pack<T, VEC>(v, p.ew.ptr[0] + off[0], p.ew.estride[0], MODE == 1);
#pragma unroll
         for (int k = 0; k < VEC; k++) part[0] = RD::combine(part[0], RD::load(v.v[k], prm));
      }
   }
   Acc acc = part[0];
#pragma unroll
   for (int u = 1; u < UNR; u++) acc = RD::combine(acc, part[u]);
   if (blockIdx.x == 0 && (int)threadIdx.x < p.ntail)
      acc = RD::combine(acc, RD::load(*reinterpret_cast<const T *>(p.tail + (int64_t)threadIdx.x * p.ew.estride[0]), prm));
   acc = block_reduce<RD, BLOCK>(acc, lds);
   if (threadIdx.x == 0)
   {  store_shared_global<Acc>(p.partials + (size_t)(p.slot_base + blockIdx.x) * OCH_RED_SLOT, acc);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");            /* the write-through stores above have completed */
      ticket = __hip_atomic_fetch_add(p.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
   }
   __syncthreads();
   if (ticket != p.total_blocks - 1) return;
   /* last block: every partial is in memory; fold them in index order */
   acc = RD::identity();
   for (unsigned int b = threadIdx.x; b < p.total_blocks; b += BLOCK)
      acc = RD::combine(acc, load_shared_global<Acc>(p.partials + (size_t)b * OCH_RED_SLOT));
   __syncthreads();
   acc = block_reduce<RD, BLOCK>(acc, lds);
   if (threadIdx.x == 0)
   {  *reinterpret_cast<typename RD::Res *>(p.result) = RD::finalize(acc, prm);
      *p.counter = 0;
   }
}


typedef int (*red_fn)(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                      const och_scalar *b1, const och_scalar *b2, double pnorm,
                      void *dresult, char *scratch, bool zero_counter, hipStream_t stream);

/* One launch: `shape` is normalised and holds at most reduce_part_limit() elements unless it is one-dimensional.
   blocks == 0: the launch stands alone and picks its own number of blocks; otherwise it is one of several that share
   the partial slots (its blocks write slots slot_base ...) and the counter (total blocks of all launches). */
template <class T, int OP>
static int launch_reduce_part(const EwShape<1> &shape, const typename Reduce<T, OP>::Param &prm, void *dresult, char *scratch,
                              unsigned int slot_base, unsigned int nblocks, unsigned int total, hipStream_t stream)
{
   typedef Reduce<T, OP> RD;
   RedParams p;
   memset(&p, 0, sizeof(p));
   constexpr int VEC = vec_for<T>();
   const int es[1] = { (int)sizeof(T) };
   bool wide_launch = false;
   if (shape.nelem > 0)
   {  if (shape.ndims == 1)
      {  uint64_t n = shape.size[0];
         constexpr size_t width = (sizeof(T) * VEC > 16) ? 16 : sizeof(T) * VEC;
         wide_launch = (n >= (uint64_t)VEC) && (shape.stride[0][0] == (int64_t)sizeof(T)) && (((uintptr_t)shape.ptr[0]) % width == 0);
         int vec = wide_launch ? VEC : 1;
         p.ew.ndims = 1; p.ew.ptr[0] = shape.ptr[0];
         p.ew.estride[0] = shape.stride[0][0]; p.ew.gstride[0] = shape.stride[0][0] * vec;
         p.ngroups = n / vec;
         p.ntail = (int)(n % vec);
         p.tail = shape.ptr[0] + (int64_t)(n - n % vec) * shape.stride[0][0];
      }
      else
      {  /* several dimensions: 128-bit loads along the first one when it is contiguous, divisible and aligned */
         wide_launch = (VEC > 1) && ew_params<1>(p.ew, shape, VEC, es, 0) && p.ew.vecmode[0] == 1;
         if (!wide_launch) ew_params<1>(p.ew, shape, 1, es, 0);
         p.ngroups = p.ew.ngroups;
      }
   }
   /* row mode: contiguous rows of at least 24 bytes that the wide path cannot take (shorter rows would load about as
      many chunks as they hold elements) */
   bool rows_launch = false;
   if constexpr (VEC > 1)
   {  if (shape.nelem > 0 && !wide_launch && shape.stride[0][0] == (int64_t)sizeof(T) && ((uintptr_t)shape.ptr[0]) % sizeof(T) == 0
          && shape.size[0] * sizeof(T) >= 24)
      {  bool ok = true;
         for (int d = 1; d < shape.ndims; d++) if (shape.stride[0][d] % (int64_t)sizeof(T) != 0) ok = false;
         const uint64_t rowbytes = shape.size[0] * sizeof(T);
         const uint64_t chunks = (16 - sizeof(T) + rowbytes + 15) / 16;            /* of the worst-placed row */
         const uint64_t rows = shape.nelem / shape.size[0];
         if (ok && chunks <= 0xFFFFFFFFull && rows * chunks <= 0xFFFF0000ull)
         {  ew_params<1>(p.ew, shape, 1, es, 0);
            p.ew.div[0] = make_fastdiv((uint32_t)chunks);
            p.rowbytes = (int64_t)rowbytes;
            p.ngroups = rows * chunks; p.ntail = 0; p.tail = nullptr;
            rows_launch = true;
         }
      }
   }
   p.partials = scratch;
   p.counter = reinterpret_cast<unsigned int *>(scratch + OCH_RED_MAX_BLOCKS * OCH_RED_SLOT);
   p.result = dresult;
   const bool streaming = wide_launch && p.ngroups * (uint64_t)(sizeof(T) * VEC) >= OCH_EW_STREAM_BYTES;
   /* Sources that are read once from memory (larger than the caches) carry the nontemporal hint (268 MB of float32
      are summed at 6.3 TB/s with it and at 5.5 TB/s without) and run as one workgroup of 512 threads per compute
      unit: every unit starts at once, works through one contiguous range with 2048 loads of 16 bytes in flight and
      hands in one partial result. Measured on 268 MB of float32 / 537 MB of float64 (GB/s): 256 x 512 threads
      6530 / 6920; 512 x 256 threads 6190 / 6800; 1024 x 256 5550 / 6450; 4096 x 256 3820 / 5540; 256 x 1024 6160 / 6580;
      eight or two loads per thread in flight instead of four 6190 / 6660 and 5080 / 5400. */
   const unsigned int threads = streaming ? OCH_RED_BLOCK_STREAM : OCH_RED_BLOCK;
   const unsigned int cap = streaming ? (unsigned int)gemm_compute_units() : OCH_RED_MAX_BLOCKS;
   uint64_t want = (p.ngroups + (uint64_t)threads * OCH_RED_UNR - 1) / ((uint64_t)threads * OCH_RED_UNR);
   unsigned int blocks = (unsigned int)(want < 1 ? 1 : (want > cap ? cap : want));
   if (blocks > OCH_RED_MAX_BLOCKS) blocks = OCH_RED_MAX_BLOCKS;
   if (nblocks != 0) blocks = nblocks;                        /* blocks beyond the data fold the identity */
   p.slot_base = slot_base; p.total_blocks = (nblocks != 0) ? total : blocks;
   {  const uint64_t step = (uint64_t)threads * OCH_RED_UNR;
      uint64_t per = (p.ngroups + blocks - 1) / blocks;
      p.per_block = (per + step - 1) / step * step;
   }
   if (streaming)        hipLaunchKernelGGL((reduce_all_kernel<RD, T, VEC, 1, true, OCH_RED_BLOCK_STREAM>), dim3(blocks), dim3(OCH_RED_BLOCK_STREAM), 0, stream, p, prm);
   else if (wide_launch) hipLaunchKernelGGL((reduce_all_kernel<RD, T, VEC, 1>), dim3(blocks), dim3(OCH_RED_BLOCK), 0, stream, p, prm);
   else if (rows_launch)
   {  if constexpr (VEC > 1) hipLaunchKernelGGL((reduce_all_kernel<RD, T, VEC, 2>), dim3(blocks), dim3(OCH_RED_BLOCK), 0, stream, p, prm); }
   else             hipLaunchKernelGGL((reduce_all_kernel<RD, T, 1, 0>),  dim3(blocks), dim3(OCH_RED_BLOCK), 0, stream, p, prm);
   OCH_CHECK_LAUNCH();
   return 0;
}

template <class T, int OP>
static int launch_reduce_all(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                             const och_scalar *b1, const och_scalar *b2, double pnorm,
                             void *dresult, char *scratch, bool zero_counter, hipStream_t stream)
{
   typedef Reduce<T, OP> RD;
   static_assert(sizeof(typename RD::Acc) <= OCH_RED_SLOT, "accumulator does not fit a partial slot");
   typename RD::Param prm;
   memset(&prm, 0, sizeof(prm));
   if (b1) memcpy(&prm.bound1, b1, sizeof(T));
   if (b2) memcpy(&prm.bound2, b2, sizeof(T));
   prm.phalf = pnorm / 2; prm.pinv = (pnorm != 0) ? 1.0 / pnorm : 0.0;

   const ptrdiff_t *st[1] = { strides }; void *pp[1] = { ptr };
   EwShape<1> shape;
   if (ew_normalize<1>(shape, ndims, size, st, pp, 0, true) != 0) return -1;
   if (shape.nelem == 0 && RD::NEEDS_DATA) return set_error("reduction of an empty tensor is undefined for this operation");
   unsigned int *counter = reinterpret_cast<unsigned int *>(scratch + OCH_RED_MAX_BLOCKS * OCH_RED_SLOT);
   if (zero_counter && fill_bytes(counter, 0, sizeof(unsigned int), stream) != 0) return -1;
   const uint64_t limit = reduce_part_limit();
   if (shape.ndims > 1 && shape.nelem > limit)
   {  /* more elements than one launch indexes: one launch per box, all of them sharing the slots and the counter */
      struct Box { uint64_t start[OCH_MAX_DIMS], count[OCH_MAX_DIMS]; };
      Box boxes[OCH_RED_MAX_PARTS];                         /* on the stack: this path allocates nothing, on the host either */
      int64_t kept = 0;
      const int64_t n = reduce_cut_parts(shape.ndims, shape.size, limit, [&](const uint64_t *start, const uint64_t *count)
                        {  if (kept < OCH_RED_MAX_PARTS)
                           {  Box &b = boxes[kept++]; for (int d = 0; d < shape.ndims; d++) { b.start[d] = start[d]; b.count[d] = count[d]; } }
                        });
      if (n < 0) return set_error("reduction: the first dimension of a strided tensor exceeds %llu elements", (unsigned long long)limit);
      if (n > OCH_RED_MAX_PARTS) return set_error("reduction: the tensor needs %lld launches, more than the %d that share the partial results", (long long)n, OCH_RED_MAX_PARTS);
      const unsigned int each = (unsigned int)(OCH_RED_MAX_PARTS / n), total = each * (unsigned int)n;
      unsigned int base = 0;
      for (int64_t k = 0; k < n; k++)
      {  const Box &b = boxes[k];
         EwShape<1> part = shape;
         int nd = 0;
         part.nelem = 1;
         for (int d = 0; d < shape.ndims; d++)
         {  part.ptr[0] += (int64_t)b.start[d] * shape.stride[0][d]; part.nelem *= b.count[d];
            if (d == 0 || b.count[d] != 1) { part.size[nd] = b.count[d]; part.stride[0][nd] = shape.stride[0][d]; nd++; }
         }
         part.ndims = nd;
         if (launch_reduce_part<T, OP>(part, prm, dresult, scratch, base, each, total, stream) != 0)
         {  /* the launches so far have drawn tickets that no later block will complete: start the next call from zero */
            (void)fill_bytes(counter, 0, sizeof(unsigned int), stream);
            return -1;
         }
         base += each;
      }
      return 0;
   }
   return launch_reduce_part<T, OP>(shape, prm, dresult, scratch, 0, 0, 0, stream);
}

template <class T, int OP, bool OK> struct PickR { static constexpr red_fn fn = nullptr; };
template <class T, int OP> struct PickR<T, OP, true> { static constexpr red_fn fn = &launch_reduce_all<T, OP>; };
template <int OP> struct RowR { static const red_fn fn[DT_COUNT]; };
#define OCH_X(T) PickR<T, OP, reduce_defined<T, OP>()>::fn,
template <int OP> const red_fn RowR<OP>::fn[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X

} /* namespace och */
