/* Compile-time construction of (operation, element type) -> launcher tables.
 * Plays the role of the LUTs that solid/bin/generate.py:236-426 writes into
 * solid_core_gpu.lut.c: a null entry means "not available for this type"
 * (checked by OC_SOLID_FUNPTR, ocean_solid.h:131-140). */
#pragma once
#include "och_elemwise.h"

namespace och {

typedef int (*ew3_fn)(int, const size_t *, const ptrdiff_t *, void *, const ptrdiff_t *, void *,
                      const ptrdiff_t *, void *, hipStream_t);
typedef int (*ew2_fn)(int, const size_t *, const ptrdiff_t *, void *, const ptrdiff_t *, void *, hipStream_t);

enum TypeSet { TS_ALL, TS_NOT_COMPLEX, TS_INT_BOOL, TS_BOOL, TS_NOT_BOOL, TS_FLOAT_COMPLEX, TS_COMPLEX, TS_NOT_UINT };

template <class T, int TS> constexpr bool in_typeset()
{
   return (TS == TS_ALL) ? true
        : (TS == TS_NOT_COMPLEX) ? !is_complex_v<T>
        : (TS == TS_INT_BOOL) ? (is_int_v<T> || is_bool_v<T>)
        : (TS == TS_BOOL) ? is_bool_v<T>
        : (TS == TS_NOT_BOOL) ? !is_bool_v<T>
        : (TS == TS_FLOAT_COMPLEX) ? (is_float_v<T> || is_complex_v<T>)
        : (TS == TS_COMPLEX) ? is_complex_v<T>
        : !is_uint_v<T>;
}

template <template <class> class OP, class T, bool OK> struct Pick3 { static constexpr ew3_fn fn = nullptr; };
template <template <class> class OP, class T> struct Pick3<OP, T, true> { static constexpr ew3_fn fn = &launch_ew3<OP<T>>; };

template <template <class> class OP, int TS> struct Row3 { static const ew3_fn fn[DT_COUNT]; };
#define OCH_X(T) Pick3<OP, T, in_typeset<T, TS>()>::fn,
template <template <class> class OP, int TS> const ew3_fn Row3<OP, TS>::fn[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X

template <class F, bool OK> struct Pick2 { static constexpr ew2_fn fn = nullptr; };
template <class F> struct Pick2<F, true> { static constexpr ew2_fn fn = &launch_ew2<F>; };

static inline int dtype_ok(int dtype) { return dtype >= 0 && dtype < DT_COUNT; }

} /* namespace och */
