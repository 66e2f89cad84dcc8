/* C ABI of the copy family: och_copy, och_byteswap_copy, och_byteswap.
 *
 * Equal shapes (after merging dimensions) go through the elementwise engine with a
 * converting functor. When the two sides have different shapes but equal element counts
 * (reshape copy, solid/src/core/gpu/template_copy.cu:35-51 / op/apply_elemwise2b.c) each
 * side is walked in its own dimension order: a size-only gather kernel handles equal
 * types directly; unequal types gather into a stream-ordered temporary in the source
 * type first and convert from there, which keeps the kernel count at one per element size
 * instead of one per type pair. */
#include "och_dispatch.h"
#include <string.h>

namespace och {
ew2_fn copy_lookup_a(int swap, int which, int dst);
ew2_fn copy_lookup_b(int swap, int which, int dst);
ew2_fn copy_lookup_c(int swap, int which, int dst);
ew2_fn copy_lookup_d(int swap, int which, int dst);
ew2_fn copy_lookup_e(int swap, int which, int dst);

static ew2_fn copy_lookup(int src, int dst, int swap)
{
   switch (src / 3)
   {  case 0: return copy_lookup_a(swap, src % 3, dst);
      case 1: return copy_lookup_b(swap, src % 3, dst);
      case 2: return copy_lookup_c(swap, src % 3, dst);
      case 3: return copy_lookup_d(swap, src % 3, dst);
      default: return copy_lookup_e(swap, src % 3, dst);
   }
}

/* ---- reshape gather: dst[flat] = src[flat], both sides strided, ES bytes per element ---- */
struct ReshapeParams
{
   char *src, *dst;
   int nd1, nd2;
   FastDiv div1[OCH_MAX_DIMS], div2[OCH_MAX_DIMS];
   int64_t st1[OCH_MAX_DIMS], st2[OCH_MAX_DIMS];
   uint32_t nelem;
};

template <int ES> struct alignas(ES) Blob { char b[ES]; };

template <int ES>
__global__ __launch_bounds__(256) void reshape_kernel(const ReshapeParams p)
{
   uint32_t e = blockIdx.x * 256 + threadIdx.x;
   if (e >= p.nelem) return;
   int64_t o1 = 0, o2 = 0;
   uint32_t q = e;
   for (int d = 0; d < p.nd1 - 1; d++) { uint32_t q2 = fastdiv(q, p.div1[d]); o1 += (int64_t)(q - q2 * p.div1[d].d) * p.st1[d]; q = q2; }
   o1 += (int64_t)q * p.st1[p.nd1 - 1];
   q = e;
   for (int d = 0; d < p.nd2 - 1; d++) { uint32_t q2 = fastdiv(q, p.div2[d]); o2 += (int64_t)(q - q2 * p.div2[d].d) * p.st2[d]; q = q2; }
   o2 += (int64_t)q * p.st2[p.nd2 - 1];
   *reinterpret_cast<Blob<ES> *>(p.dst + o2) = *reinterpret_cast<const Blob<ES> *>(p.src + o1);
}

struct Side { int nd; uint64_t size[OCH_MAX_DIMS]; int64_t st[OCH_MAX_DIMS]; uint64_t nelem; };

/* drop unit dimensions and merge adjacent mergeable ones, keeping the order */
static int side_normalize(Side &s, int ndims, const size_t *size, const ptrdiff_t *strides)
{
   if (ndims < 0 || ndims > OCH_MAX_DIMS) return set_error("invalid number of dimensions (%d)", ndims);
   s.nd = 0; s.nelem = 1;
   for (int d = 0; d < ndims; d++)
   {  s.nelem *= size[d];
      if (size[d] == 1) continue;
      if (s.nd > 0 && strides[d] == s.st[s.nd - 1] * (int64_t)s.size[s.nd - 1]) s.size[s.nd - 1] *= size[d];
      else { s.size[s.nd] = size[d]; s.st[s.nd] = strides[d]; s.nd++; }
   }
   if (s.nd == 0) { s.nd = 1; s.size[0] = 1; s.st[0] = 0; }
   return 0;
}

/* the same for element counts above the launch limit of the elementwise engine: sizes and the flat index are 64 bits
   wide and decomposed with plain divisions; one launch covers elements [first, first + count) */
struct ReshapeBigParams
{
   char *src, *dst;
   int nd1, nd2;
   uint64_t size1[OCH_MAX_DIMS], size2[OCH_MAX_DIMS];
   int64_t st1[OCH_MAX_DIMS], st2[OCH_MAX_DIMS];
   uint64_t first, count;
};
template <int ES>
__global__ __launch_bounds__(256) void reshape_big_kernel(const ReshapeBigParams p)
{
   const uint64_t local = (uint64_t)blockIdx.x * 256 + threadIdx.x;
   if (local >= p.count) return;
   const uint64_t e = p.first + local;
   int64_t o1 = 0, o2 = 0;
   uint64_t q = e;
   for (int d = 0; d < p.nd1 - 1; d++) { const uint64_t q2 = q / p.size1[d]; o1 += (int64_t)(q - q2 * p.size1[d]) * p.st1[d]; q = q2; }
   o1 += (int64_t)q * p.st1[p.nd1 - 1];
   q = e;
   for (int d = 0; d < p.nd2 - 1; d++) { const uint64_t q2 = q / p.size2[d]; o2 += (int64_t)(q - q2 * p.size2[d]) * p.st2[d]; q = q2; }
   o2 += (int64_t)q * p.st2[p.nd2 - 1];
   *reinterpret_cast<Blob<ES> *>(p.dst + o2) = *reinterpret_cast<const Blob<ES> *>(p.src + o1);
}

static int reshape_launch(int es, const Side &a, char *src, const Side &b, char *dst, hipStream_t stream)
{
   if (a.nelem > ew_launch_limit())
   {  /* the two sides are cut differently by their dimensions, so the cut is made along the flat index they share
         (the reference runs its kernel with 64-bit indices, solid/src/core/gpu/op/apply_elemwise.c:66-99) */
      ReshapeBigParams p;
      p.src = src; p.dst = dst; p.nd1 = a.nd; p.nd2 = b.nd;
      for (int d = 0; d < a.nd; d++) { p.size1[d] = a.size[d]; p.st1[d] = a.st[d]; }
      for (int d = 0; d < b.nd; d++) { p.size2[d] = b.size[d]; p.st2[d] = b.st[d]; }
      const uint64_t run = ew_launch_limit();
      for (uint64_t first = 0; first < a.nelem; first += run)
      {  p.first = first; p.count = (a.nelem - first < run) ? a.nelem - first : run;
         dim3 grid((unsigned)((p.count + 255) / 256)), block(256);
         switch (es)
         {  case 1:  hipLaunchKernelGGL(reshape_big_kernel<1>,  grid, block, 0, stream, p); break;
            case 2:  hipLaunchKernelGGL(reshape_big_kernel<2>,  grid, block, 0, stream, p); break;
            case 4:  hipLaunchKernelGGL(reshape_big_kernel<4>,  grid, block, 0, stream, p); break;
            case 8:  hipLaunchKernelGGL(reshape_big_kernel<8>,  grid, block, 0, stream, p); break;
            default: hipLaunchKernelGGL(reshape_big_kernel<16>, grid, block, 0, stream, p); break;
         }
         OCH_CHECK_LAUNCH();
      }
      return 0;
   }
   ReshapeParams p;
   p.src = src; p.dst = dst; p.nd1 = a.nd; p.nd2 = b.nd; p.nelem = (uint32_t)a.nelem;
   for (int d = 0; d < a.nd; d++) { p.div1[d] = make_fastdiv((uint32_t)a.size[d]); p.st1[d] = a.st[d]; }
   for (int d = 0; d < b.nd; d++) { p.div2[d] = make_fastdiv((uint32_t)b.size[d]); p.st2[d] = b.st[d]; }
   dim3 grid((p.nelem + 255) / 256), block(256);
   switch (es)
   {  case 1:  hipLaunchKernelGGL(reshape_kernel<1>,  grid, block, 0, stream, p); break;
      case 2:  hipLaunchKernelGGL(reshape_kernel<2>,  grid, block, 0, stream, p); break;
      case 4:  hipLaunchKernelGGL(reshape_kernel<4>,  grid, block, 0, stream, p); break;
      case 8:  hipLaunchKernelGGL(reshape_kernel<8>,  grid, block, 0, stream, p); break;
      default: hipLaunchKernelGGL(reshape_kernel<16>, grid, block, 0, stream, p); break;
   }
   OCH_CHECK_LAUNCH();
   return 0;
}

static int copy_impl(int ts, int td, int swap,
                     int nd1, const size_t *size1, const ptrdiff_t *st1, void *p1,
                     int nd2, const size_t *size2, const ptrdiff_t *st2, void *p2, hipStream_t stream)
{
   if (!dtype_ok(ts) || !dtype_ok(td)) return set_error("invalid data type (%d, %d)", ts, td);
   {  /* equal shapes: the elementwise engine merges the dimensions of both sides together (merging each side on its own
         would give a transposed source and a dense destination different shapes and send them down the reshape path) */
      bool same = (nd1 == nd2) && nd1 >= 0 && nd1 <= OCH_MAX_DIMS;
      for (int d = 0; d < nd1 && same; d++) same = (size1[d] == size2[d]);
      if (same) return copy_lookup(ts, td, swap)(nd1, size1, st1, p1, st2, p2, stream);
   }
   Side a, b;
   if (side_normalize(a, nd1, size1, st1) != 0 || side_normalize(b, nd2, size2, st2) != 0) return -1;
   if (a.nelem != b.nelem) return set_error("copy: element counts differ (%llu, %llu)", (unsigned long long)a.nelem, (unsigned long long)b.nelem);
   if (a.nelem == 0) return 0;
   bool regular = (a.nd == b.nd);
   for (int d = 0; d < a.nd && regular; d++) regular = (a.size[d] == b.size[d]);
   if (regular)
   {  size_t sz[OCH_MAX_DIMS]; ptrdiff_t s1[OCH_MAX_DIMS], s2[OCH_MAX_DIMS];
      for (int d = 0; d < a.nd; d++) { sz[d] = a.size[d]; s1[d] = a.st[d]; s2[d] = b.st[d]; }
      return copy_lookup(ts, td, swap)(a.nd, sz, s1, p1, s2, p2, stream);
   }
   int es = och_type_size[ts];
   if (ts == td && !swap) return reshape_launch(es, a, (char *)p1, b, (char *)p2, stream);
   /* gather into a contiguous temporary of the source type, then convert with the destination's shape */
   void *tmp = nullptr;
   OCH_CHECK_HIP(hipMallocAsync(&tmp, a.nelem * es, stream));
   Side flat; flat.nd = 1; flat.size[0] = a.nelem; flat.st[0] = es; flat.nelem = a.nelem;
   int status = reshape_launch(es, a, (char *)p1, flat, (char *)tmp, stream);
   if (status == 0)
   {  size_t sz[OCH_MAX_DIMS]; ptrdiff_t s1[OCH_MAX_DIMS], s2[OCH_MAX_DIMS]; int64_t acc = es;
      for (int d = 0; d < b.nd; d++) { sz[d] = b.size[d]; s1[d] = acc; acc *= (int64_t)b.size[d]; s2[d] = b.st[d]; }
      status = copy_lookup(ts, td, swap)(b.nd, sz, s1, tmp, s2, p2, stream);
   }
   (void)hipFreeAsync(tmp, stream);
   return status;
}

/* in-place byte reversal of every real part */
template <class T> struct SwapInPlace
{  typedef T R; struct Param {}; static constexpr bool RMW = true;
   static OCH_D R f(R x, uint64_t, const Param &) { return byteswap<T>(x); }
};
typedef int (*ew1_swap_fn)(int, const size_t *, const ptrdiff_t *, void *, hipStream_t);
template <class T> static int launch_swap(int nd, const size_t *size, const ptrdiff_t *st, void *ptr, hipStream_t stream)
{  typename SwapInPlace<T>::Param prm; return launch_ew1<SwapInPlace<T>>(nd, size, st, ptr, prm, true, stream); }
#define OCH_X(T) &launch_swap<T>,
static const ew1_swap_fn swap_table[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X
}

extern "C" int och_copy(int dtype_src, int dtype_dst,
                        int ndims1, const size_t *size1, const ptrdiff_t *strides1, void *ptr1,
                        int ndims2, const size_t *size2, const ptrdiff_t *strides2, void *ptr2, och_stream stream)
{  return och::copy_impl(dtype_src, dtype_dst, 0, ndims1, size1, strides1, ptr1, ndims2, size2, strides2, ptr2, och::as_stream(stream)); }

extern "C" int och_byteswap_copy(int dtype_src, int dtype_dst,
                        int ndims1, const size_t *size1, const ptrdiff_t *strides1, void *ptr1,
                        int ndims2, const size_t *size2, const ptrdiff_t *strides2, void *ptr2, och_stream stream)
{  return och::copy_impl(dtype_src, dtype_dst, 1, ndims1, size1, strides1, ptr1, ndims2, size2, strides2, ptr2, och::as_stream(stream)); }

extern "C" int och_byteswap(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, och_stream stream)
{
   if (!och::dtype_ok(dtype)) return och::set_error("invalid data type (%d)", dtype);
   if (och_type_size[dtype] == 1 || dtype == OCH_BOOL) return 0;           /* one-byte parts: nothing to do */
   return och::swap_table[dtype](ndims, size, strides, ptr, och::as_stream(stream));
}
