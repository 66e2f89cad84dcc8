/* Axis reductions for gfx950: dst[outer] = reduce over the reduced dimensions of src.
 *
 * Replaces the three kernel modes of solid/include/solid/core/gpu/reduce_axis.h:142-597 and
 * their host-side planner (solid/src/core/gpu/op/reduce_axis.c:22-315). Two kernel shapes:
 *   thread-per-output  : neighbouring threads own neighbouring outputs; used when the outer
 *                        dimension is the fast one in memory, so every load instruction of a
 *                        wave is contiguous; eight loads in flight per thread, and four waves
 *                        share each group of 64 outputs when there are few outputs
 *   group-per-output   : a wave (64) or a block (256) strides over the reduced range of one
 *                        output and combines with a shuffle butterfly (+ LDS for blocks); used
 *                        when the reduced dimension is the fast one in memory
 * Accumulator types, NaN rules and result types are those of the full reductions.
 */
#pragma once
#include <vector>
#include "och_reduce_all.h"

namespace och {

struct AxisParams
{
   char    *src, *dst;
   int      nd, rd;
   FastDiv  div[OCH_MAX_DIMS], rdiv[OCH_MAX_DIMS];
   uint32_t glanes;                              /* lanes per output in the wave-cooperative kernel */
   uint32_t opb;                                 /* output groups per block in the sharing per-thread kernel */
   /* few outputs, long reduced range: grid y cuts the reduced range into `slices` pieces of slice_len (rows of the
      reduced range when slice_rows is set, else positions along its first dimension; the cooperative kernels count in
      loads); every piece leaves its accumulator in partials[slice][output] (16-byte slots) and axis_finish_kernel
      folds the pieces in order */
   uint32_t slices, slice_len; int slice_rows;
   /* partial: the accumulators go to partials[slice_base + slice][output] instead of the destination (always when the
      range is cut into slices; also for a single slice when the call is one of several that cover a reduced range too
      long for one launch, whose pieces occupy consecutive slots and are folded together) */
   int partial; uint32_t slice_base;
   int64_t  rowbytes;                            /* row mode of the cooperative kernels: bytes of one row of the first reduced dimension */
   /* row mode of the per-thread kernel: the rows of the first outer dimension are not whole aligned groups, but every row
      starts at the same position row_m within a 16-byte unit; a thread owns the aligned chunk c of a row, i.e. the
      outputs c * VEC - row_m / sizeof(T) + k that lie inside the row (rgdiv: chunks per row) */
   uint32_t row_groups, row_n0; int row_m;
   int      dst_wide;                            /* per-thread kernel: the VEC results of a thread are neighbours in memory and 16-byte aligned */
   char    *partials;
   FastDiv  rgdiv;                               /* 128-bit groups per row of the first reduced dimension (cooperative kernels) */
   int64_t  st1[OCH_MAX_DIMS], st2[OCH_MAX_DIMS], rst[OCH_MAX_DIMS];
   uint32_t nout, relem, rsize0, rrows;          /* relem = rsize0 * rrows */
};

OCH_D void axis_outer_offsets(const AxisParams &p, uint32_t o, int64_t &o1, int64_t &o2)
{
   o1 = 0; o2 = 0;
   uint32_t q = o;
   for (int d = 0; d < p.nd - 1; d++)
   {  uint32_t q2 = fastdiv(q, p.div[d]); uint32_t i = q - q2 * p.div[d].d; q = q2;
      o1 += (int64_t)i * p.st1[d]; o2 += (int64_t)i * p.st2[d];
   }
   if (p.nd > 0) { o1 += (int64_t)q * p.st1[p.nd - 1]; o2 += (int64_t)q * p.st2[p.nd - 1]; }
}

/* offset of row r of the reduced range (all reduced dimensions but the first) */
OCH_D int64_t axis_row_offset(const AxisParams &p, uint32_t r)
{
   int64_t off = 0; uint32_t q = r;
   for (int d = 1; d < p.rd - 1; d++)
   {  uint32_t q2 = fastdiv(q, p.rdiv[d]); off += (int64_t)(q - q2 * p.rdiv[d].d) * p.rst[d]; q = q2; }
   if (p.rd > 1) off += (int64_t)q * p.rst[p.rd - 1];
   return off;
}

/* Workgroups are dealt to the 8 XCDs round-robin, each XCD with its own L2. This permutation of the block index
   (within runs of 32 blocks) gives every XCD 4 consecutive logical blocks, so that blocks working on neighbouring
   segments of the same rows -- which share the cache lines at the segment boundaries when the row pitch is not a
   multiple of the line size -- meet in one L2 instead of fetching those lines from memory twice. */
OCH_D uint32_t xcd_neighbour_block(uint32_t b, uint32_t nblocks)
{  const uint32_t chunk = b & ~31u, r = b & 31u;
   if (chunk + 32 > nblocks) return b;
   return chunk + (r & 7u) * 4 + (r >> 3);
}

/* Neighbouring threads own neighbouring outputs: VEC consecutive outputs each (one 128-bit load
   covers them; needs unit source stride along the first outer dimension). SPLIT slices (waves
   when SPLIT is 4) share each output: slice s takes elements s, s + SPLIT, ... of every row of
   the reduced range and the slices are folded through LDS in slice order. */
template <class RD, class T, int SPLIT, int VEC, bool NT = false, bool ROWS = false>
__global__ __launch_bounds__(256) void axis_thread_kernel(const AxisParams p, const typename RD::Param prm)
{
   typedef typename RD::Acc Acc;
   /* output groups per block: 256 without sharing; with sharing p.opb (a power of two, at most 128: fewer when there are
      fewer groups, so that the lanes of a wave still read neighbouring memory), the other 256 / p.opb threads of a group
      being its slices */
   const uint32_t OPB = (SPLIT > 1) ? p.opb : 256u, NSL = 256u / OPB;
   constexpr int UNR = (VEC > 1) ? 4 : 8;
   __shared__ Acc lds[SPLIT > 1 ? 256 * VEC : 1];
   const uint32_t slice = threadIdx.x / OPB, ol = threadIdx.x % OPB;
   const uint32_t group = xcd_neighbour_block(blockIdx.x, gridDim.x) * OPB + ol;
   /* first output of the thread; row mode: first output of the thread's row, and the position of pack element 0 in it */
   uint32_t o = group * VEC; int first = 0; int64_t chunk = 0;
   bool active = o < p.nout;
   if constexpr (ROWS)
   {  active = group < p.row_groups;
      const uint32_t q = fastdiv(group, p.rgdiv), c = group - q * p.rgdiv.d;
      o = q * p.row_n0;
      first = (int)(c * VEC) - p.row_m / (int)sizeof(T);
      chunk = (int64_t)c * 16 - p.row_m;
   }
   Acc acc[VEC];
#pragma unroll
   for (int k = 0; k < VEC; k++) acc[k] = RD::identity();
   int64_t o1 = 0, o2 = 0;
   if (active)
   {  axis_outer_offsets(p, o, o1, o2);
      const char *base = p.src + o1 + chunk;
      const int64_t s0 = p.rst[0];
      uint32_t r_lo = 0, r_hi = p.rrows, i_lo = 0, i_hi = p.rsize0;
      if (p.slices > 1)
      {  const uint32_t a = blockIdx.y * p.slice_len;
         if (p.slice_rows) { r_lo = a; r_hi = (a + p.slice_len < p.rrows) ? a + p.slice_len : p.rrows; }
         else { i_lo = a; i_hi = (a + p.slice_len < p.rsize0) ? a + p.slice_len : p.rsize0; }
      }
      for (uint32_t r = r_lo; r < r_hi; r++)
      {  const char *row = base + ((p.rd > 1) ? axis_row_offset(p, r) : 0);
         uint32_t i = i_lo + slice;
         for (; i + (UNR - 1) * NSL < i_hi; i += UNR * NSL)
         {  Pack<T, VEC> v[UNR];
#pragma unroll
            for (int u = 0; u < UNR; u++) load_wide<T, VEC, NT>(v[u], row + (int64_t)(i + u * NSL) * s0);
#pragma unroll
            for (int u = 0; u < UNR; u++)
#pragma unroll
               for (int k = 0; k < VEC; k++) acc[k] = RD::combine(acc[k], RD::load(v[u].v[k], prm));
         }
         for (; i < i_hi; i += NSL)
         {  Pack<T, VEC> v;
            load_wide<T, VEC>(v, row + (int64_t)i * s0);
#pragma unroll
            for (int k = 0; k < VEC; k++) acc[k] = RD::combine(acc[k], RD::load(v.v[k], prm));
         }
      }
   }
   if constexpr (SPLIT > 1)
   {
#pragma unroll
      for (int k = 0; k < VEC; k++) lds[k * 256 + threadIdx.x] = acc[k];
      __syncthreads();
      if (slice == 0)
      {
         for (uint32_t s2 = 1; s2 < NSL; s2++)
#pragma unroll
            for (int k = 0; k < VEC; k++) acc[k] = RD::combine(acc[k], lds[k * 256 + s2 * OPB + ol]);
      }
   }
   if (active && slice == 0)
   {  typedef typename RD::Res Res;
      /* results per store instruction: up to 16 bytes. Element-wise stores of a thread's VEC results put the lanes of
         one store instruction VEC results apart (sums of 2 x 2^25 int8 into int64: 1.8 TB/s). */
      constexpr int PV = (VEC > 1) ? ((sizeof(Res) * VEC >= 16) ? (int)(16 / sizeof(Res)) : VEC) : 1;
      if constexpr (ROWS)
      {
#pragma unroll
         for (int k = 0; k < VEC; k++)
         {  const int i = first + k;                   /* position in the row; elements of the chunk outside the row are dropped */
            if (i >= 0 && (uint32_t)i < p.row_n0)
            {  if (p.partial) *reinterpret_cast<Acc *>(p.partials + ((size_t)(p.slice_base + blockIdx.y) * p.nout + o + (uint32_t)i) * 16) = acc[k];
               else *reinterpret_cast<Res *>(p.dst + o2 + (int64_t)i * p.st2[0]) = RD::finalize(acc[k], prm);
            }
         }
      }
      else if (VEC > 1 && p.dst_wide && !p.partial)
      {
#pragma unroll
         for (int q = 0; q < VEC / PV; q++)
         {  Pack<Res, PV> out;
#pragma unroll
            for (int k = 0; k < PV; k++) out.v[k] = RD::finalize(acc[q * PV + k], prm);
            store_wide<Res, PV>(out, p.dst + o2 + (int64_t)(q * PV) * (int64_t)sizeof(Res));
         }
      }
      else
      {
#pragma unroll
         for (int k = 0; k < VEC; k++)
         {  if (p.partial) *reinterpret_cast<Acc *>(p.partials + ((size_t)(p.slice_base + blockIdx.y) * p.nout + o + k) * 16) = acc[k];
            else *reinterpret_cast<Res *>(p.dst + o2 + (int64_t)k * p.st2[0]) = RD::finalize(acc[k], prm);
         }
      }
   }
}

/* folds the pieces of a sliced reduction: `lanes` threads (a power of two, at most 64) per output. A lane takes pieces
   lane, lane + lanes, ... in that order, four loads in flight, and the lanes are combined by a butterfly: a fixed order
   for a given number of pieces, so the result is reproducible. With one thread per output the fold of a thousand pieces
   was a chain of a thousand dependent memory latencies and took longer than the reduction itself. */
template <class RD, class T>
__global__ __launch_bounds__(256) void axis_finish_kernel(const AxisParams p, const typename RD::Param prm, const uint32_t lanes)
{
   typedef typename RD::Acc Acc;
   const uint32_t o = (blockIdx.x * 256 + threadIdx.x) / lanes, lane = threadIdx.x % lanes;
   const bool active = o < p.nout;
   Acc acc = RD::identity();
   if (active)
   {  const char *slot = p.partials + (size_t)o * 16;
      const size_t pitch = (size_t)p.nout * 16;
      uint32_t t = lane;
      for (; t + 3 * lanes < p.slices; t += 4 * lanes)
      {  Acc v[4];
#pragma unroll
         for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const Acc *>(slot + (size_t)(t + u * lanes) * pitch);
#pragma unroll
         for (int u = 0; u < 4; u++) acc = RD::combine(acc, v[u]);
      }
      for (; t < p.slices; t += lanes) acc = RD::combine(acc, *reinterpret_cast<const Acc *>(slot + (size_t)t * pitch));
   }
#pragma unroll
   for (int m = 32; m >= 1; m >>= 1) if ((uint32_t)m < lanes) acc = RD::combine(acc, shfl_xor_any<Acc>(acc, m));
   if (active && lane == 0)
   {  int64_t o1, o2;
      axis_outer_offsets(p, o, o1, o2);
      *reinterpret_cast<typename RD::Res *>(p.dst + o2) = RD::finalize(acc, prm);
   }
}

/* One load of the cooperative kernels: element (VEC 1), aligned 16-byte group i of the row (VEC > 1), or -- row mode,
   for contiguous rows that are not whole aligned groups: odd width, odd pitch, a start inside a 16-byte unit -- the
   aligned 16-byte chunk i counted from the row start rounded down to 16, of which only the elements [lo, hi) belong
   to the row. A chunk is loaded only when it holds an element of the row. */
template <class T, int VEC, bool ROWS, bool NT>
OCH_D void axis_fetch(Pack<T, VEC> &v, const char *rowbase, uint32_t i, int64_t s0, int64_t rowbytes, int &lo, int &hi)
{
   if constexpr (VEC > 1 && ROWS)
   {  const int64_t first = (int64_t)i * 16 - (int64_t)((uintptr_t)rowbase & 15);
      const int64_t left = rowbytes - first;
      lo = (first < 0) ? (int)((-first) / (int64_t)sizeof(T)) : 0;
      hi = (left <= 0) ? 0 : ((left >= 16) ? VEC : (int)(left / (int64_t)sizeof(T)));
      if (hi > lo) load_wide<T, VEC>(v, rowbase + first);
   }
   else if constexpr (VEC > 1) { lo = 0; hi = VEC; load_wide<T, VEC, NT>(v, rowbase + (int64_t)i * s0); }
   else { lo = 0; hi = 1; v.v[0] = *reinterpret_cast<const T *>(rowbase + (int64_t)i * s0); }
}

/* A group of threads cooperates on one output: GROUP 256 = the whole block, GROUP 64 = p.glanes (8 .. 64, a power
   of two) lanes of a wave (1 .. 64), chosen so that every lane has about four loads in flight on short rows. VEC > 1: the first reduced
   dimension has unit stride and every row starts 16-byte aligned, so a thread takes VEC neighbouring elements with
   one 128-bit load (NT: with the nontemporal hint, for sources that are read once from memory); ROWS: see axis_fetch. */
template <class RD, class T, int GROUP, int VEC = 1, bool NT = false, bool ROWS = false>
__global__ __launch_bounds__(256) void axis_group_kernel(const AxisParams p, const typename RD::Param prm)
{
   typedef typename RD::Acc Acc;
   __shared__ Acc lds[4];
   const uint32_t G = (GROUP == 256) ? 256u : p.glanes;
   const uint32_t lane = threadIdx.x % G;
   const uint32_t o = blockIdx.x * (256 / G) + threadIdx.x / G;
   const bool active = o < p.nout;
   Acc acc = RD::identity();
   int64_t o1 = 0, o2 = 0;
   if (active)
   {  axis_outer_offsets(p, o, o1, o2);
      const char *base = p.src + o1;
      const int64_t s0 = (VEC > 1) ? (int64_t)(sizeof(T) * VEC) : p.rst[0];        /* step of one group */
      const uint32_t n0 = (VEC > 1) ? p.rgdiv.d : p.rsize0;                        /* groups (chunks) per row */
      /* range of loads of this piece of the reduced range */
      const uint32_t total = (p.rd <= 1) ? n0 : ((VEC > 1) ? p.rrows * n0 : p.relem);
      uint32_t lo = 0, hi = total;
      if (p.slices > 1) { lo = blockIdx.y * p.slice_len; hi = (lo + p.slice_len < total) ? lo + p.slice_len : total; }
      if (p.rd <= 1)
      {  uint32_t i = lo + lane;
         for (; i + 3 * G < hi; i += 4 * G)
         {  Pack<T, VEC> v[4]; int klo[4], khi[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
            {  if constexpr (ROWS) v[u] = Pack<T, VEC>{};
               axis_fetch<T, VEC, ROWS, NT>(v[u], base, i + u * G, s0, p.rowbytes, klo[u], khi[u]);
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
               for (int k = 0; k < VEC; k++) if (k >= klo[u] && k < khi[u]) acc = RD::combine(acc, RD::load(v[u].v[k], prm));
         }
         for (; i < hi; i += G)
         {  Pack<T, VEC> v; int klo, khi;
            if constexpr (ROWS) v = Pack<T, VEC>{};
            axis_fetch<T, VEC, ROWS, NT>(v, base, i, s0, p.rowbytes, klo, khi);
#pragma unroll
            for (int k = 0; k < VEC; k++) if (k >= klo && k < khi) acc = RD::combine(acc, RD::load(v.v[k], prm));
         }
      }
      else
      {  for (uint32_t j = lo + lane; j < hi; j += G)
         {  uint32_t r = fastdiv(j, (VEC > 1) ? p.rgdiv : p.rdiv[0]); uint32_t i = j - r * n0;
            Pack<T, VEC> v; int klo, khi;
            if constexpr (ROWS) v = Pack<T, VEC>{};
            axis_fetch<T, VEC, ROWS, NT>(v, base + axis_row_offset(p, r), i, s0, p.rowbytes, klo, khi);
#pragma unroll
            for (int k = 0; k < VEC; k++) if (k >= klo && k < khi) acc = RD::combine(acc, RD::load(v.v[k], prm));
         }
      }
   }
#pragma unroll
   for (int m = 32; m >= 1; m >>= 1) if (GROUP == 256 || (uint32_t)m < G) acc = RD::combine(acc, shfl_xor_any<Acc>(acc, m));
   if constexpr (GROUP == 256)
   {  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
      __syncthreads();
      if (threadIdx.x == 0) { acc = RD::combine(RD::combine(lds[0], lds[1]), RD::combine(lds[2], lds[3])); }
   }
   if (active && lane == 0)
   {  if (p.partial) *reinterpret_cast<Acc *>(p.partials + ((size_t)(p.slice_base + blockIdx.y) * p.nout + o) * 16) = acc;
      else *reinterpret_cast<typename RD::Res *>(p.dst + o2) = RD::finalize(acc, prm);
   }
}

/* Short contiguous rows (one reduced dimension of 1 ... 64 aligned 16-byte groups, a power of two of them): p.glanes =
   groups per row lanes share an output, every lane loads ONE group per output, and a lane group takes four outputs, one
   per load instruction, so that each instruction of a wave reads 1 KB of consecutive rows and four are in flight. With one
   output per lane group a lane had a single load in flight (rows of two groups), or read its row's groups one after the
   other from lines it shared with its neighbours (8 floats per output: 5.3 TB/s). */
template <class RD, class T, int VEC, bool NT>
__global__ __launch_bounds__(256) void axis_short_rows_kernel(const AxisParams p, const typename RD::Param prm)
{
   typedef typename RD::Acc Acc;
   constexpr int U = 4;
   const uint32_t G = p.glanes, gpw = 64u / G;
   const uint32_t wave = (blockIdx.x * 256u + threadIdx.x) >> 6, lane = threadIdx.x & 63u, g = lane / G, li = lane % G;
   Pack<T, VEC> v[U]; int64_t o2[U]; bool active[U];
#pragma unroll
   for (int u = 0; u < U; u++)
   {  const uint32_t o = (wave * U + u) * gpw + g;
      active[u] = o < p.nout;
      int64_t o1 = 0; o2[u] = 0;
      if (active[u])
      {  axis_outer_offsets(p, o, o1, o2[u]);
         load_wide<T, VEC, NT>(v[u], p.src + o1 + (int64_t)li * 16);
      }
   }
#pragma unroll
   for (int u = 0; u < U; u++)
   {  Acc acc = RD::identity();
      if (active[u])
      {
#pragma unroll
         for (int k = 0; k < VEC; k++) acc = RD::combine(acc, RD::load(v[u].v[k], prm));
      }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) if ((uint32_t)m < G) acc = RD::combine(acc, shfl_xor_any<Acc>(acc, m));
      if (active[u] && li == 0) *reinterpret_cast<typename RD::Res *>(p.dst + o2[u]) = RD::finalize(acc, prm);
   }
}

typedef int (*axis_fn)(const och_reduce_axis_config *c, double pnorm);
/* outputs one launch handles (0xFFFFFF00 unless och_reduce_axis_set_output_limit has lowered it for a test) */
uint64_t axis_output_limit();
/* elements of the reduced range (per output) one launch handles: 0xFFFFFF00 unless och_reduce_axis_set_range_limit has
   lowered it for a test */
uint64_t axis_range_limit();

/* One launch of several that together cover a reduced range too long for one: it leaves its accumulators in the slots
   base, base + 1, ... of the stream's workspace (at most `room` of them) and reports how many it used. */
struct AxisPiece { uint32_t base, room, used; AxisParams params; };

/* Cuts the reduced range of c into pieces of at most `limit` elements, in the order of the flat reduced index: runs
   along the outermost reduced dimension, or -- when a single index of it is still too long -- index by index, each cut
   further inside. */
static void axis_cut_range(const och_reduce_axis_config &c, uint64_t limit, std::vector<och_reduce_axis_config> &out)
{
   uint64_t relem = 1; int last = -1;
   for (int d = 0; d < c.rdims; d++) { relem *= c.rsize[d]; if (c.rsize[d] > 1) last = d; }
   if (relem <= limit || last < 0) { out.push_back(c); return; }
   const uint64_t inner = relem / c.rsize[last];
   if (inner <= limit)
   {  const uint64_t run = limit / inner;
      for (uint64_t start = 0; start < c.rsize[last]; start += run)
      {  och_reduce_axis_config piece = c;
         piece.rsize[last] = (c.rsize[last] - start < run) ? (size_t)(c.rsize[last] - start) : (size_t)run;
         piece.ptr1 = (char *)c.ptr1 + (int64_t)start * c.rstrides[last];
         out.push_back(piece);
      }
      return;
   }
   for (uint64_t i = 0; i < c.rsize[last]; i++)
   {  och_reduce_axis_config piece = c;
      piece.rsize[last] = 1;
      piece.ptr1 = (char *)c.ptr1 + (int64_t)i * c.rstrides[last];
      axis_cut_range(piece, limit, out);
   }
}

template <class T, int OP>
static int launch_reduce_axis_one(const och_reduce_axis_config *c, const typename Reduce<T, OP>::Param &prm,
                                  uint64_t nout, uint64_t relem, AxisPiece *piece);

template <class T, int OP>
static int launch_reduce_axis(const och_reduce_axis_config *c, double pnorm)
{
   typedef Reduce<T, OP> RD;
   if (c->ndims < 0 || c->ndims > OCH_MAX_DIMS || c->rdims < 0 || c->rdims > OCH_MAX_DIMS)
      return set_error("invalid number of dimensions (%d, %d)", c->ndims, c->rdims);
   typename RD::Param prm;
   memset(&prm, 0, sizeof(prm));
   prm.phalf = pnorm / 2; prm.pinv = (pnorm != 0) ? 1.0 / pnorm : 0.0;
   uint64_t nout = 1, relem = 1;
   for (int d = 0; d < c->ndims; d++) nout *= c->size[d];
   for (int d = 0; d < c->rdims; d++) relem *= c->rsize[d];
   if (nout == 0) return 0;
   if (relem == 0 && RD::NEEDS_DATA) return set_error("reduction over an empty range is undefined for this operation");
   /* more outputs than one launch counts in 32 bits (the reference switches to 64-bit indices): the outputs are
      independent, so the outermost kept dimension is cut into runs that fit, or walked index by index when a single
      index of it is still too much, and every piece is a reduction of its own on the same stream */
   if (nout > axis_output_limit())
   {  int last = -1;
      for (int d = 0; d < c->ndims; d++) if (c->size[d] > 1) last = d;
      const uint64_t inner = nout / c->size[last];
      const uint64_t run = (inner <= axis_output_limit()) ? axis_output_limit() / inner : 1;
      for (uint64_t start = 0; start < c->size[last]; start += run)
      {  och_reduce_axis_config piece = *c;
         piece.size[last] = (c->size[last] - start < run) ? (size_t)(c->size[last] - start) : (size_t)run;
         piece.ptr1 = (char *)c->ptr1 + (int64_t)start * c->strides1[last];
         piece.ptr2 = (char *)c->ptr2 + (int64_t)start * c->strides2[last];
         if (launch_reduce_axis<T, OP>(&piece, pnorm) != 0) return -1;
      }
      return 0;
   }
   if (relem <= axis_range_limit()) return launch_reduce_axis_one<T, OP>(c, prm, nout, relem, nullptr);
   /* a reduced range longer than one launch counts in 32 bits (solid/src/core/gpu/op/apply_elemwise.c:66-99: the
      reference switches to 64-bit indices): the range is cut into pieces, every piece is a launch that leaves raw
      accumulators in consecutive slots of the stream's workspace -- cut into slices of its own while there is room -- and
      one finish kernel folds all slots in the order of the reduced index */
   std::vector<och_reduce_axis_config> pieces;
   axis_cut_range(*c, axis_range_limit(), pieces);
   const uint64_t rows = OCH_GEMM_WORKSPACE / (nout * 16);
   if (pieces.size() > rows) return set_error("axis reduction: the reduced range needs %llu pieces of partial results, the workspace holds %llu",
                                              (unsigned long long)pieces.size(), (unsigned long long)rows);
   AxisPiece pc; uint32_t base = 0;
   for (size_t i = 0; i < pieces.size(); i++)
   {  uint64_t n = 1;
      for (int d = 0; d < pieces[i].rdims; d++) n *= pieces[i].rsize[d];
      pc.base = base; pc.used = 0;
      pc.room = (uint32_t)(rows - base - (pieces.size() - 1 - i));           /* every later piece needs at least one slot */
      if (launch_reduce_axis_one<T, OP>(&pieces[i], prm, nout, n, &pc) != 0) return -1;
      base += pc.used;
   }
   AxisParams p = pc.params;
   p.slices = base; p.slice_base = 0;
   uint32_t lanes = 1;
   while (lanes < 64 && lanes * 16 <= p.slices && (uint64_t)p.nout * lanes * 2 <= (1u << 20)) lanes *= 2;
   hipLaunchKernelGGL((axis_finish_kernel<RD, T>), dim3((unsigned)(((uint64_t)p.nout * lanes + 255) / 256)), dim3(256), 0, as_stream(c->stream), p, prm, lanes);
   OCH_CHECK_LAUNCH();
   return 0;
}

template <class T, int OP>
static int launch_reduce_axis_one(const och_reduce_axis_config *c, const typename Reduce<T, OP>::Param &prm,
                                  uint64_t nout, uint64_t relem, AxisPiece *piece)
{
   typedef Reduce<T, OP> RD;
   AxisParams p;
   memset(&p, 0, sizeof(p));
   p.src = (char *)c->ptr1; p.dst = (char *)c->ptr2;
   /* drop unit dimensions */
   for (int d = 0; d < c->ndims; d++)
   {  if (c->size[d] == 1) continue;
      p.div[p.nd] = make_fastdiv((uint32_t)c->size[d]); p.st1[p.nd] = c->strides1[d]; p.st2[p.nd] = c->strides2[d]; p.nd++;
   }
   uint64_t rs0 = 1;
   for (int d = 0; d < c->rdims; d++)
   {  if (c->rsize[d] == 1) continue;
      if (p.rd == 0) rs0 = c->rsize[d];
      p.rdiv[p.rd] = make_fastdiv((uint32_t)c->rsize[d]); p.rst[p.rd] = c->rstrides[d]; p.rd++;
   }
   p.nout = (uint32_t)nout; p.relem = (uint32_t)relem;
   p.rsize0 = (relem == 0) ? 0 : (uint32_t)rs0;
   p.rrows = (relem == 0) ? 0 : (uint32_t)(relem / rs0);
   hipStream_t stream = as_stream(c->stream);

   /* which side is the fast one in memory? */
   int64_t outer_fast = (p.nd > 0) ? (p.st1[0] < 0 ? -p.st1[0] : p.st1[0]) : INT64_MAX;
   for (int d = 1; d < p.nd; d++) { int64_t a = p.st1[d] < 0 ? -p.st1[d] : p.st1[d]; if (a < outer_fast) outer_fast = a; }
   int64_t red_fast = (p.rd > 0) ? (p.rst[0] < 0 ? -p.rst[0] : p.rst[0]) : INT64_MAX;
   /* a source larger than the caches is read once: nontemporal loads (see och_reduce_all.h) */
   const bool streaming = nout * relem * (uint64_t)sizeof(T) >= OCH_EW_STREAM_BYTES;
   /* cooperate on an output when the reduced range is the faster one in memory (or there is a single output); otherwise
      neighbouring threads take neighbouring outputs, and a long reduced range is cut into pieces below */
   bool cooperative = (p.rd > 0) && ((red_fast < outer_fast) || p.nd == 0);
   /* too few blocks for the device and a long reduced range: cut the range into pieces (grid y), about 1024 blocks in all,
      every piece at least min_len long, the partial accumulators within the stream's workspace */
   auto plan_slices = [&](uint64_t blocks, uint64_t range, uint64_t min_len) -> int
   {  p.slices = 1; p.slice_len = 0; p.partials = nullptr;
      p.partial = piece ? 1 : 0; p.slice_base = piece ? piece->base : 0;
      if (blocks < 512 && range >= 2 * min_len)
      {  uint64_t want = (1024 + blocks - 1) / blocks;
         if (want > range / min_len) want = range / min_len;
         const uint64_t fit = piece ? (uint64_t)piece->room : OCH_GEMM_WORKSPACE / ((uint64_t)p.nout * 16);
         if (want > fit) want = fit;
         if (want > 65535) want = 65535;
         if (want >= 2)
         {  p.slice_len = (uint32_t)((range + want - 1) / want);
            p.slices = (uint32_t)((range + p.slice_len - 1) / p.slice_len);
            if (p.slices < 2) p.slices = 1;
         }
      }
      if (p.slices > 1) p.partial = 1;
      return p.partial ? stream_gemm_workspace(stream, &p.partials) : 0;
   };
   if (!cooperative)
   {  /* VEC outputs per thread when the first outer dimension has unit source stride and
         everything is 16-byte aligned; four waves per output group while there are few groups */
      constexpr int VEC = vec_for<T>();
      bool wide = (VEC > 1) && p.nd > 0 && p.st1[0] == (int64_t)sizeof(T) && (p.div[0].d % VEC == 0) && (((uintptr_t)p.src) % 16 == 0);
      for (int d = 1; d < p.nd && wide; d++) if (p.st1[d] % 16 != 0) wide = false;
      for (int d = 0; d < p.rd && wide; d++) if (p.rst[d] % 16 != 0) wide = false;
      p.dst_wide = (wide && p.st2[0] == (int64_t)sizeof(typename RD::Res) && (((uintptr_t)p.dst) % 16 == 0)) ? 1 : 0;
      for (int d = 1; d < p.nd && p.dst_wide; d++) if (p.st2[d] % 16 != 0) p.dst_wide = 0;
      /* row mode: unit stride along the first outer dimension, every other stride a multiple of 16 bytes (so all rows
         start at the same position within a 16-byte unit), rows of at least 24 bytes, but not whole aligned groups */
      bool rows = false;
      if (VEC > 1 && !wide && p.nd > 0 && p.st1[0] == (int64_t)sizeof(T) && ((uintptr_t)p.src) % sizeof(T) == 0 && (uint64_t)p.div[0].d * sizeof(T) >= 24)
      {  rows = true;
         for (int d = 1; d < p.nd; d++) if (p.st1[d] % 16 != 0) rows = false;
         for (int d = 0; d < p.rd; d++) if (p.rst[d] % 16 != 0) rows = false;
         if (rows)
         {  p.row_m = (int)(((uintptr_t)p.src) % 16); p.row_n0 = p.div[0].d;
            const uint64_t chunks = ((uint64_t)p.row_m + (uint64_t)p.row_n0 * sizeof(T) + 15) / 16;
            const uint64_t total = chunks * (nout / p.row_n0);
            if (total > 0xFFFFFF00ull) rows = false;
            else { p.rgdiv = make_fastdiv((uint32_t)chunks); p.row_groups = (uint32_t)total; }
         }
      }
      const uint64_t groups = wide ? nout / VEC : (rows ? (uint64_t)p.row_groups : nout);
      const bool split = groups < (1u << 20) && p.rsize0 >= 16;
      p.opb = 64;
      /* four or more blocks per compute unit: twice the outputs per block and half the slices (float64 512 x 512 x 256
         reduced along its second dimension: 1024 blocks of 64 groups 6.2-6.3 TB/s, 512 blocks of 128 groups 6.7) */
      if (split && wide && groups / 64 >= 4 * (uint64_t)gemm_compute_units()) p.opb = 128;
      while (p.opb > 1 && p.opb / 2 >= groups) p.opb /= 2;
      /* fewer blocks than compute units: narrower blocks (down to 32 groups = 512 contiguous bytes per row) before the
         reduced range is cut into pieces, which costs a second kernel */
      if (split && wide) while (p.opb > 32 && (groups + p.opb - 1) / p.opb < 256 && p.rsize0 >= 32 * (256 / (p.opb / 2))) p.opb /= 2;
      const unsigned blocks = (unsigned)(split ? (groups + p.opb - 1) / p.opb : (groups + 255) / 256);
      /* pieces of the reduced range: whole rows of it when there are several, else positions along its first dimension */
      p.slice_rows = (p.rd > 1 && p.rrows >= 8) ? 1 : 0;
      if (plan_slices(blocks, p.slice_rows ? p.rrows : p.rsize0, p.slice_rows ? 4 : (split ? 16 * (256 / p.opb) : 16)) != 0) return -1;
      const dim3 grid(blocks, p.slices);
      if (wide && split && streaming) hipLaunchKernelGGL((axis_thread_kernel<RD, T, 4, VEC, true>), grid, dim3(256), 0, stream, p, prm);
      else if (wide && split)         hipLaunchKernelGGL((axis_thread_kernel<RD, T, 4, VEC>), grid, dim3(256), 0, stream, p, prm);
      else if (wide && streaming)     hipLaunchKernelGGL((axis_thread_kernel<RD, T, 1, VEC, true>), grid, dim3(256), 0, stream, p, prm);
      else if (wide)                  hipLaunchKernelGGL((axis_thread_kernel<RD, T, 1, VEC>), grid, dim3(256), 0, stream, p, prm);
      else if (rows)
      {  if constexpr (VEC > 1)
         {  if (split) hipLaunchKernelGGL((axis_thread_kernel<RD, T, 4, VEC, false, true>), grid, dim3(256), 0, stream, p, prm);
            else       hipLaunchKernelGGL((axis_thread_kernel<RD, T, 1, VEC, false, true>), grid, dim3(256), 0, stream, p, prm);
         }
      }
      else if (split)                 hipLaunchKernelGGL((axis_thread_kernel<RD, T, 4, 1>), grid, dim3(256), 0, stream, p, prm);
      else                            hipLaunchKernelGGL((axis_thread_kernel<RD, T, 1, 1>), grid, dim3(256), 0, stream, p, prm);
   }
   else
   {  /* rows of the first reduced dimension are contiguous and 16-byte aligned: 128-bit loads */
      constexpr int VEC = vec_for<T>();
      bool wide = (VEC > 1) && p.rst[0] == (int64_t)sizeof(T) && (p.rsize0 % VEC == 0) && (((uintptr_t)p.src) % 16 == 0);
      for (int d = 0; d < p.nd && wide; d++) if (p.st1[d] % 16 != 0) wide = false;
      for (int d = 1; d < p.rd && wide; d++) if (p.rst[d] % 16 != 0) wide = false;
      if (wide) p.rgdiv = make_fastdiv(p.rsize0 / VEC);
      /* row mode: contiguous rows of at least 24 bytes that are not whole aligned groups */
      bool rows = false;
      if (VEC > 1 && !wide && p.rst[0] == (int64_t)sizeof(T) && ((uintptr_t)p.src) % sizeof(T) == 0 && (uint64_t)p.rsize0 * sizeof(T) >= 24)
      {  rows = true;
         for (int d = 0; d < p.nd; d++) if (p.st1[d] % (int64_t)sizeof(T) != 0) rows = false;
         for (int d = 1; d < p.rd; d++) if (p.rst[d] % (int64_t)sizeof(T) != 0) rows = false;
         const uint64_t rowbytes = (uint64_t)p.rsize0 * sizeof(T);
         const uint64_t chunks = (16 - sizeof(T) + rowbytes + 15) / 16;             /* of the worst-placed row */
         if (chunks * p.rrows > 0xFFFFFF00ull) rows = false;
         if (rows) { p.rgdiv = make_fastdiv((uint32_t)chunks); p.rowbytes = (int64_t)rowbytes; }
      }
      const bool wave = relem <= 2048 && nout >= 1024;              /* a wave per output, else a block per output */
      const uint32_t loads = wide ? p.relem / VEC : (rows ? p.rrows * p.rgdiv.d : p.relem);       /* loads per output: about four per lane */
      p.glanes = 64;
      while (p.glanes > 1 && (p.glanes / 2) * 4 >= loads) p.glanes /= 2;
      const uint32_t per_block = 256 / p.glanes;
      const unsigned blocks = wave ? (p.nout + per_block - 1) / per_block : p.nout;
      p.slice_rows = 0;
      {  const uint64_t range = (p.rd <= 1) ? (wide ? p.rsize0 / VEC : (rows ? p.rgdiv.d : p.rsize0)) : loads;
         if (plan_slices(blocks, range, (uint64_t)(wave ? p.glanes : 256) * 8) != 0) return -1;
      }
      /* short rows: one load per lane and output, four outputs per lane group (see axis_short_rows_kernel) */
      if (VEC > 1 && wide && wave && p.rd == 1 && p.slices == 1 && !p.partial && loads <= 64 && (loads & (loads - 1)) == 0)
      {  if constexpr (VEC > 1)
         {  p.glanes = loads;
            const uint64_t waves = ((uint64_t)p.nout + 4 * (64 / loads) - 1) / (4 * (64 / loads));
            const unsigned sblocks = (unsigned)((waves + 3) / 4);
            if (streaming) hipLaunchKernelGGL((axis_short_rows_kernel<RD, T, VEC, true>), dim3(sblocks), dim3(256), 0, stream, p, prm);
            else           hipLaunchKernelGGL((axis_short_rows_kernel<RD, T, VEC, false>), dim3(sblocks), dim3(256), 0, stream, p, prm);
            OCH_CHECK_LAUNCH();
            return 0;
         }
      }
      const dim3 grid(blocks, p.slices);
      /* the nontemporal hint only where one load instruction of a wave covers whole cache lines: with fewer than eight
         lanes per output the four loads of a lane share their lines with its neighbours' loads, and lines that are not
         kept came from memory twice (8 floats per output: 3.8 TB/s with the hint) */
      if (wide && streaming && (!wave || p.glanes >= 8))
      {  if (wave) hipLaunchKernelGGL((axis_group_kernel<RD, T, 64, VEC, true>), grid, dim3(256), 0, stream, p, prm);
         else      hipLaunchKernelGGL((axis_group_kernel<RD, T, 256, VEC, true>), grid, dim3(256), 0, stream, p, prm);
      }
      else if (wide)
      {  if (wave) hipLaunchKernelGGL((axis_group_kernel<RD, T, 64, VEC>), grid, dim3(256), 0, stream, p, prm);
         else      hipLaunchKernelGGL((axis_group_kernel<RD, T, 256, VEC>), grid, dim3(256), 0, stream, p, prm);
      }
      else if (rows)
      {  if constexpr (VEC > 1)
         {  if (wave) hipLaunchKernelGGL((axis_group_kernel<RD, T, 64, VEC, false, true>), grid, dim3(256), 0, stream, p, prm);
            else      hipLaunchKernelGGL((axis_group_kernel<RD, T, 256, VEC, false, true>), grid, dim3(256), 0, stream, p, prm);
         }
      }
      else
      {  if (wave) hipLaunchKernelGGL((axis_group_kernel<RD, T, 64>), grid, dim3(256), 0, stream, p, prm);
         else      hipLaunchKernelGGL((axis_group_kernel<RD, T, 256>), grid, dim3(256), 0, stream, p, prm);
      }
   }
   if (piece) { OCH_CHECK_LAUNCH(); piece->used = p.slices; piece->params = p; return 0; }
   if (p.slices > 1)
   {  uint32_t lanes = 1;                        /* at least eight pieces per lane, at most 2^20 threads */
      while (lanes < 64 && lanes * 16 <= p.slices && (uint64_t)p.nout * lanes * 2 <= (1u << 20)) lanes *= 2;
      hipLaunchKernelGGL((axis_finish_kernel<RD, T>), dim3((unsigned)(((uint64_t)p.nout * lanes + 255) / 256)), dim3(256), 0, stream, p, prm, lanes);
   }
   OCH_CHECK_LAUNCH();
   return 0;
}

template <class T, int OP, bool OK> struct PickA { static constexpr axis_fn fn = nullptr; };
template <class T, int OP> struct PickA<T, OP, true> { static constexpr axis_fn fn = &launch_reduce_axis<T, OP>; };
template <int OP> struct RowA { static const axis_fn fn[DT_COUNT]; };
#define OCH_X(T) PickA<T, OP, reduce_defined<T, OP>()>::fn,
template <int OP> const axis_fn RowA<OP>::fn[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X

} /* namespace och */
