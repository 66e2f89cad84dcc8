/* Fill, conditional fill and steps (the reference's elemwise1 family:
 * solid/src/core/gpu/template_fill.cu:35-82, template_steps.cu:31-57; CPU semantics
 * solid/src/core/cpu/template_fill.c:30-60, template_steps.c:31-100). */
#include "och_dispatch.h"
#include "och_ops_unary.h"
#include <string.h>

namespace och {

template <class T> struct FillOp
{  typedef T R; struct Param { T value; }; static constexpr bool RMW = false;
   static OCH_D R f(R, uint64_t, const Param &p) { return p.value; }
};
template <class T> struct FillNaNOp
{  typedef T R; struct Param { T value; }; static constexpr bool RMW = true;
   static OCH_D R f(R x, uint64_t, const Param &p) { return fillnan_test<T>(x) ? p.value : x; }
};

/* value = offset + index * step in the arithmetic of the parameter type, converted to the
   work type and then to the element type. With 64-bit integer parameters the index is an
   unsigned 64-bit value, so the sum is formed modulo 2^64 and converted as unsigned. */
template <class T, class V> OCH_D T steps_store(V v)
{
   if constexpr (is_bool_v<T>)
   {  T r;
      if constexpr (std::is_same<V, double>::value) r.v = float_to_int<uint8_t, double>(v); else r.v = (uint8_t)v;
      return r;
   }
   else if constexpr (is_complex_v<T>)
   {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W;
      T r; r.real = from_work<E>(cvt_real<W, V>(v)); r.imag = from_work<E>((W)0); return r;
   }
   else { typedef typename traits<T>::work W; return from_work<T>(cvt_real<W, V>(v)); }
}
template <class T> struct StepsInt64Op
{  typedef T R; struct Param { int64_t offset, step; }; static constexpr bool RMW = false;
   static OCH_D R f(R, uint64_t i, const Param &p) { return steps_store<T, uint64_t>((uint64_t)p.offset + i * (uint64_t)p.step); }
};
template <class T> struct StepsDoubleOp
{  typedef T R; struct Param { double offset, step; }; static constexpr bool RMW = false;
   static OCH_D R f(R, uint64_t i, const Param &p) { return steps_store<T, double>(p.offset + (double)i * p.step); }
};
template <class T> struct StepsCDoubleOp
{  typedef T R; struct Param { double ro, io, rs, is; }; static constexpr bool RMW = false;
   static OCH_D R f(R, uint64_t i, const Param &p)
   {  if constexpr (is_complex_v<T>)
      {  typedef typename traits<T>::elem E; typedef elemwork_t<T> W; T r;
         r.real = from_work<E>(cvt_real<W, double>(p.ro + (double)i * p.rs));
         r.imag = from_work<E>(cvt_real<W, double>(p.io + (double)i * p.is));
         return r;
      }
      else return steps_store<T, double>(p.ro + (double)i * p.rs);
   }
};

template <class T> static T scalar_as(const och_scalar &s) { T v; memcpy(&v, &s, sizeof(T)); return v; }

template <template <class> class OP, class T>
static int launch_fill(int nd, const size_t *size, const ptrdiff_t *st, void *ptr, const och_scalar &value, hipStream_t stream)
{  typename OP<T>::Param prm; prm.value = scalar_as<T>(value);
   return launch_ew1<OP<T>>(nd, size, st, ptr, prm, true, stream);
}
typedef int (*fill_fn)(int, const size_t *, const ptrdiff_t *, void *, const och_scalar &, hipStream_t);
#define OCH_X(T) &launch_fill<FillOp, T>,
static const fill_fn fill_table[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X
static const fill_fn fillnan_table[DT_COUNT] = { 0, 0, 0, 0, 0, 0, 0, 0, 0,
   &launch_fill<FillNaNOp, half_t>, &launch_fill<FillNaNOp, float>, &launch_fill<FillNaNOp, double>,
   &launch_fill<FillNaNOp, chalf_t>, &launch_fill<FillNaNOp, cfloat_t>, &launch_fill<FillNaNOp, cdouble_t> };

/* ---- masked fill: data[i] = value where mask[i] ----
   A thread owns VEC neighbouring elements (16 bytes of the tensor, VEC mask bytes). Where the tensor is unit-stride and
   aligned, the group moves as a whole: nothing when no mask byte of the group is set, one 16-byte store when all are,
   otherwise the group is read, the set elements are replaced and the group is written back -- stores of single
   elements leave the memory system to merge them into the lines it holds, which runs at about half the rate. Otherwise
   element by element. */
template <class T, int VEC>
__global__ __launch_bounds__(OCH_EW_BLOCK) void masked_fill_kernel(const EwParams<2> p, const T value)
{
   uint32_t g = blockIdx.x * OCH_EW_BLOCK + threadIdx.x;
   if (g >= p.ngroups) return;
   int64_t off[2];
   group_offsets<2>(p, g, off);
   Pack<obool, VEC> m;
   load_pack<obool, VEC>(m, p.ptr[1] + off[1], p.estride[1], p.vecmode[1]);
   if (VEC > 1 && p.vecmode[0] == 1)
   {  bool any = false, all = true;
#pragma unroll
      for (int k = 0; k < VEC; k++) { any = any || (m.v[k].v != 0); all = all && (m.v[k].v != 0); }
      if (!any) return;
      Pack<T, VEC> d;
      if (!all) load_wide<T, VEC>(d, p.ptr[0] + off[0]);
#pragma unroll
      for (int k = 0; k < VEC; k++) if (all || m.v[k].v) d.v[k] = value;
      store_wide<T, VEC>(d, p.ptr[0] + off[0]);
      return;
   }
#pragma unroll
   for (int k = 0; k < VEC; k++)
      if (m.v[k].v) *reinterpret_cast<T *>(p.ptr[0] + off[0] + k * p.estride[0]) = value;
}
template <class T>
static int launch_masked_fill(int nd, const size_t *size, const ptrdiff_t *st1, void *p1, const ptrdiff_t *st2, void *p2,
                              const och_scalar &value, hipStream_t stream)
{
   const ptrdiff_t *strides[2] = { st1, st2 }; void *ptrs[2] = { p1, p2 };
   EwShape<2> shape;
   if (ew_normalize<2>(shape, nd, size, strides, ptrs, 0, true) != 0) return -1;
   const int es[2] = { (int)sizeof(T), 1 };
   T v = scalar_as<T>(value);
   constexpr int VEC = vec_for<T>();
   return ew_launch_chunked<2>(shape, 0, [&](const EwShape<2> &s, uint64_t flat0) -> int
   {  EwParams<2> p;
      if (VEC > 1 && ew_params<2>(p, s, VEC, es, flat0))
         hipLaunchKernelGGL((masked_fill_kernel<T, VEC>), dim3((p.ngroups + OCH_EW_BLOCK - 1) / OCH_EW_BLOCK), dim3(OCH_EW_BLOCK), 0, stream, p, v);
      else
      {  ew_params<2>(p, s, 1, es, flat0);
         hipLaunchKernelGGL((masked_fill_kernel<T, 1>), dim3((p.ngroups + OCH_EW_BLOCK - 1) / OCH_EW_BLOCK), dim3(OCH_EW_BLOCK), 0, stream, p, v);
      }
      OCH_CHECK_LAUNCH();
      return 0;
   });
}
typedef int (*mfill_fn)(int, const size_t *, const ptrdiff_t *, void *, const ptrdiff_t *, void *, const och_scalar &, hipStream_t);
#define OCH_X(T) &launch_masked_fill<T>,
static const mfill_fn mfill_table[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X

}  /* namespace och */

using namespace och;

extern "C" int och_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, och_scalar value, och_stream stream)
{
   if (!dtype_ok(dtype)) return set_error("invalid data type (%d)", dtype);
   return fill_table[dtype](ndims, size, strides, ptr, value, as_stream(stream));
}
extern "C" int och_fill_nan(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, och_scalar value, och_stream stream)
{
   if (!dtype_ok(dtype) || fillnan_table[dtype] == 0) return set_error("fill_nan is not available for data type %d", dtype);
   return fillnan_table[dtype](ndims, size, strides, ptr, value, as_stream(stream));
}
extern "C" int och_masked_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides1, void *ptr1,
                               const ptrdiff_t *strides2, void *ptr2, och_scalar value, och_stream stream)
{
   if (!dtype_ok(dtype)) return set_error("invalid data type (%d)", dtype);
   return mfill_table[dtype](ndims, size, strides1, ptr1, strides2, ptr2, value, as_stream(stream));
}

extern "C" int och_steps_int64(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                               int64_t offset, int64_t step, och_stream stream)
{
   switch (dtype)
   {
#define OCH_X(T) case traits<T>::index: { StepsInt64Op<T>::Param prm; prm.offset = offset; prm.step = step; \
                    return launch_ew1<StepsInt64Op<T>>(ndims, size, strides, ptr, prm, false, as_stream(stream)); }
      OCH_FOR_ALL_TYPES(OCH_X)
#undef OCH_X
   }
   return set_error("invalid data type (%d)", dtype);
}
extern "C" int och_steps_double(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                                double offset, double step, och_stream stream)
{
   switch (dtype)
   {
#define OCH_X(T) case traits<T>::index: { StepsDoubleOp<T>::Param prm; prm.offset = offset; prm.step = step; \
                    return launch_ew1<StepsDoubleOp<T>>(ndims, size, strides, ptr, prm, false, as_stream(stream)); }
      OCH_FOR_ALL_TYPES(OCH_X)
#undef OCH_X
   }
   return set_error("invalid data type (%d)", dtype);
}
extern "C" int och_steps_cdouble(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                                 och_cdouble offset, och_cdouble step, och_stream stream)
{
   switch (dtype)
   {
#define OCH_X(T) case traits<T>::index: { StepsCDoubleOp<T>::Param prm; prm.ro = offset.real; prm.io = offset.imag; \
                    prm.rs = step.real; prm.is = step.imag; \
                    return launch_ew1<StepsCDoubleOp<T>>(ndims, size, strides, ptr, prm, false, as_stream(stream)); }
      OCH_FOR_ALL_TYPES(OCH_X)
#undef OCH_X
   }
   return set_error("invalid data type (%d)", dtype);
}
