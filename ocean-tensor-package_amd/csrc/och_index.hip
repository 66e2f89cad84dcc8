/* Index operations: add-if-negative, index-to-offset, gather / scatter / fill through per-dimension
 * offset tables. Replaces solid/src/core/gpu/template_index.cu:37-200 and the kernels of
 * solid/include/solid/core/gpu/index1.h:182-215, index2.h:188-230.
 *
 * Offset tables: for dimension d, offsets[d] is either NULL (the element offset advances by
 * index * strides[d]) or a device array of size[d] byte offsets. Gather, scatter and fill move
 * raw elements, so one kernel per element size serves every data type.
 */
#include "och_elemwise.h"
#include "och_dispatch.h"

namespace och {

template <class T> struct AddIfNegOp
{  typedef T R; struct Param { T value; }; static constexpr bool RMW = true;
   static OCH_D R f(R x, uint64_t, const Param &p) { return (x < 0) ? (R)(x + p.value) : x; }
};
template <class T> static T idx_scalar_as(const och_scalar &s) { T v; memcpy(&v, &s, sizeof(T)); return v; }

struct IndexParams
{
   uint64_t       size[OCH_MAX_DIMS];
   FastDiv        div[OCH_MAX_DIMS];           /* used when nelem < 2^32 */
   const int64_t *offsets[OCH_MAX_DIMS];
   int64_t        strides1[OCH_MAX_DIMS], strides2[OCH_MAX_DIMS];
   char          *ptr1, *ptr2;
   uint64_t       nelem;
   int            ndims;
   int            small;                       /* nelem fits one launch's 32-bit index arithmetic: div[] is filled */
};
struct ToOffsetStrides { int64_t s[OCH_MAX_DIMS]; };

template <class T>
__global__ __launch_bounds__(256) void index_to_offset_kernel(uint64_t nelem, int nstrides, const ToOffsetStrides st,
      int64_t stride_reduce, const char *src, int64_t stride1, char *dst, int64_t stride2)
{
   uint64_t j = (uint64_t)blockIdx.x * 256 + threadIdx.x;
   if (j >= nelem) return;
   int64_t s = 0;
   for (int i = 0; i < nstrides; i++)
      s += st.s[i] * (int64_t)*reinterpret_cast<const T *>(src + (int64_t)j * stride1 + (int64_t)i * stride_reduce);
   *reinterpret_cast<int64_t *>(dst + (int64_t)j * stride2) = s;
}

/* MODE 0: gather  *ptr2 = *ptr1(indexed);  1: scatter  *ptr1(indexed) = *ptr2;  2: fill  *ptr1(indexed) = value.
   V > 1: a work item is a run of V elements (16 bytes) along a dense dimension 0 that has no offset table; the host has
   divided size[0] by V and set both strides of dimension 0 to 16. Offset tables are device data, so whether a run is
   16-byte aligned is only known here: aligned runs move in one access, others element by element. */
template <class E, int MODE, int V, bool NT = false>
__global__ __launch_bounds__(256) void index_kernel(const IndexParams p, const E value)
{
   const bool small = p.small != 0;
   for (uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x; idx < p.nelem; idx += (uint64_t)gridDim.x * 256)
   {  int64_t o1 = 0, o2 = 0;
      if (small)
      {  uint32_t q = (uint32_t)idx;
         for (int d = 0; d < p.ndims; d++)
         {  const uint32_t q2 = fastdiv(q, p.div[d]), s = q - q2 * p.div[d].d; q = q2;
            o1 += p.offsets[d] ? p.offsets[d][s] : (int64_t)s * p.strides1[d];
            if (MODE != 2) o2 += (int64_t)s * p.strides2[d];
         }
      }
      else
      {  uint64_t q = idx;
         for (int d = 0; d < p.ndims; d++)
         {  uint64_t s = q % p.size[d]; q /= p.size[d];
            o1 += p.offsets[d] ? p.offsets[d][s] : (int64_t)s * p.strides1[d];
            if (MODE != 2) o2 += (int64_t)s * p.strides2[d];
         }
      }
      char *a = p.ptr1 + o1, *b = p.ptr2 + o2;
      if (V > 1 && ((((uintptr_t)a) | (MODE != 2 ? (uintptr_t)b : 0)) & 15) == 0)
      {  typedef typename RawVec<16>::type W;
         if constexpr (NT && MODE != 2)
         {  if (MODE == 0) __builtin_nontemporal_store(__builtin_nontemporal_load(reinterpret_cast<const W *>(a)), reinterpret_cast<W *>(b));
            else           *reinterpret_cast<W *>(a) = *reinterpret_cast<const W *>(b);
         }
         else if (MODE == 0) *reinterpret_cast<uint4 *>(b) = *reinterpret_cast<const uint4 *>(a);
         else if (MODE == 1) *reinterpret_cast<uint4 *>(a) = *reinterpret_cast<const uint4 *>(b);
         else { union { uint4 w; E e[V]; } u; for (int k = 0; k < V; k++) u.e[k] = value; *reinterpret_cast<uint4 *>(a) = u.w; }
         continue;
      }
      for (int k = 0; k < V; k++)
      {  E *x = reinterpret_cast<E *>(a) + k;
         if (MODE == 0) reinterpret_cast<E *>(b)[k] = *x;
         else if (MODE == 1) *x = reinterpret_cast<const E *>(b)[k];
         else *x = value;
      }
   }
}

struct alignas(4) E4 { unsigned char b[4]; };
struct alignas(8) E8 { unsigned char b[8]; };
struct alignas(8) E16 { unsigned char b[16]; };      /* cdouble is 8-byte aligned */
struct alignas(2) E2 { unsigned char b[2]; };
struct E1 { unsigned char b[1]; };

template <class E, int MODE>
static int launch_index(IndexParams &p, const och_scalar &value, hipStream_t stream)
{  E v; memcpy(&v, &value, sizeof(E));
   constexpr int V = 16 / (int)sizeof(E);
   const bool runs = p.ndims >= 1 && p.offsets[0] == nullptr && p.size[0] % V == 0 && p.strides1[0] == (int64_t)sizeof(E) &&
                     (MODE == 2 || p.strides2[0] == (int64_t)sizeof(E));
   if (runs) { p.size[0] /= V; p.nelem /= V; p.strides1[0] = 16; if (MODE != 2) p.strides2[0] = 16; }
   /* above the launch limit of the elementwise engine (2^32 - 2^16 elements unless a test has lowered it) the kernel
      decomposes the 64-bit work-item number with plain divisions; its grid-stride loop covers any count */
   p.small = (p.nelem <= ew_launch_limit()) ? 1 : 0;
   /* the call moves more than the caches hold: 16-byte runs with the nontemporal hint (a compile-time property of the kernel) */
   const bool nt = runs && MODE == 0 && p.nelem * 32 >= OCH_EW_STREAM_BYTES;      /* gathers only: scattered rows are written faster by plain stores */
   if (p.small)
      for (int d = 0; d < p.ndims; d++) p.div[d] = make_fastdiv((uint32_t)p.size[d]);
   uint64_t blocks = (p.nelem + 255) / 256; if (blocks > (1u << 20)) blocks = 1u << 20;
   if (nt)   hipLaunchKernelGGL((index_kernel<E, MODE, V, true>), dim3((unsigned)blocks), dim3(256), 0, stream, p, v);
   else if (runs) hipLaunchKernelGGL((index_kernel<E, MODE, V>), dim3((unsigned)blocks), dim3(256), 0, stream, p, v);
   else      hipLaunchKernelGGL((index_kernel<E, MODE, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, p, v);
   OCH_CHECK_LAUNCH();
   return 0;
}

template <int MODE>
static int index_op(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                    const ptrdiff_t *strides2, void *ptr2, const och_scalar &value, hipStream_t stream)
{
   if (!dtype_ok(dtype)) return set_error("invalid data type (%d)", dtype);
   if (ndims < 0 || ndims > OCH_MAX_DIMS) return set_error("invalid number of dimensions (%d)", ndims);
   IndexParams p; memset(&p, 0, sizeof(p));
   p.ndims = ndims; p.nelem = 1; p.ptr1 = (char *)ptr1; p.ptr2 = (char *)ptr2;
   for (int d = 0; d < ndims; d++)
   {  p.size[d] = size[d]; p.nelem *= size[d];
      p.offsets[d] = offsets ? offsets[d] : nullptr;
      p.strides1[d] = strides1 ? strides1[d] : 0;
      p.strides2[d] = (MODE != 2 && strides2) ? strides2[d] : 0;
   }
   if (p.nelem == 0) return 0;
   switch (och_type_size[dtype])
   {  case 1:  return launch_index<E1, MODE>(p, value, stream);
      case 2:  return launch_index<E2, MODE>(p, value, stream);
      case 4:  return launch_index<E4, MODE>(p, value, stream);
      case 8:  return launch_index<E8, MODE>(p, value, stream);
      case 16: return launch_index<E16, MODE>(p, value, stream);
   }
   return set_error("unsupported element size");
}

} /* namespace och */

using namespace och;

extern "C" int och_add_if_negative(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                                   och_scalar value, och_stream stream)
{
   switch (dtype)
   {
#define OCH_CASE(T, ID) case ID: { AddIfNegOp<T>::Param prm; prm.value = idx_scalar_as<T>(value); \
                        return launch_ew1<AddIfNegOp<T>>(ndims, size, strides, ptr, prm, true, as_stream(stream)); }
      OCH_CASE(int8_t, OCH_INT8) OCH_CASE(int16_t, OCH_INT16) OCH_CASE(int32_t, OCH_INT32) OCH_CASE(int64_t, OCH_INT64)
#undef OCH_CASE
   }
   return set_error("add_if_negative is available for signed integer types only (got %d)", dtype);
}

extern "C" int och_index_to_offset(int dtype, int nstrides, const int64_t *strides, ptrdiff_t stride_reduce, size_t nelem,
                                   ptrdiff_t stride1, void *ptr1, ptrdiff_t stride2, void *ptr2, och_stream stream)
{
   if (nstrides < 0 || nstrides > OCH_MAX_DIMS) return set_error("invalid number of strides (%d)", nstrides);
   if (nelem == 0) return 0;
   ToOffsetStrides st; memset(&st, 0, sizeof(st));
   for (int i = 0; i < nstrides; i++) st.s[i] = strides[i];
   /* launches of at most 2^31 elements each (the grid of one launch is 32 bits of blocks wide, and the runtime accepts
      far fewer blocks than that), or of the launch limit of the elementwise engine when a test has lowered it */
   const size_t per_launch = (ew_launch_limit() < ((size_t)1 << 31)) ? (size_t)ew_launch_limit() : ((size_t)1 << 31);
   for (size_t first = 0; first < nelem; first += per_launch)
   {  const size_t n = (nelem - first < per_launch) ? nelem - first : per_launch;
      const dim3 grid((unsigned)((n + 255) / 256)), block(256);
      const char *src = (const char *)ptr1 + (int64_t)first * (int64_t)stride1;
      char *dst = (char *)ptr2 + (int64_t)first * (int64_t)stride2;
      switch (dtype)
      {
#define OCH_CASE(T, ID) case ID: hipLaunchKernelGGL((index_to_offset_kernel<T>), grid, block, 0, as_stream(stream), (uint64_t)n, nstrides, st, \
                           (int64_t)stride_reduce, src, (int64_t)stride1, dst, (int64_t)stride2); break;
         OCH_CASE(uint8_t, OCH_UINT8) OCH_CASE(uint16_t, OCH_UINT16) OCH_CASE(uint32_t, OCH_UINT32) OCH_CASE(uint64_t, OCH_UINT64)
         OCH_CASE(int8_t, OCH_INT8) OCH_CASE(int16_t, OCH_INT16) OCH_CASE(int32_t, OCH_INT32) OCH_CASE(int64_t, OCH_INT64)
#undef OCH_CASE
         default: return set_error("index_to_offset is available for integer types only (got %d)", dtype);
      }
      OCH_CHECK_LAUNCH();
   }
   return 0;
}

extern "C" int och_get_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                             const ptrdiff_t *strides2, void *ptr2, och_stream stream)
{  och_scalar zero; memset(&zero, 0, sizeof(zero));
   return index_op<0>(dtype, ndims, size, offsets, strides1, ptr1, strides2, ptr2, zero, as_stream(stream));
}
extern "C" int och_set_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                             const ptrdiff_t *strides2, void *ptr2, och_stream stream)
{  och_scalar zero; memset(&zero, 0, sizeof(zero));
   return index_op<1>(dtype, ndims, size, offsets, strides1, ptr1, strides2, ptr2, zero, as_stream(stream));
}
extern "C" int och_fill_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides, void *ptr,
                              och_scalar value, och_stream stream)
{  return index_op<2>(dtype, ndims, size, offsets, strides, ptr, nullptr, nullptr, value, as_stream(stream)); }
