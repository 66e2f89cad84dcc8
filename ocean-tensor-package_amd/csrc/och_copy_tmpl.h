/* Converting copy functors and their launcher rows.
 * CvtOp<S, D, SWAP>: y = (D) x, with the source element byte-reversed part by part first
 * when SWAP is set (SOLID_ASSIGN / SOLID_BYTESWAP_ASSIGN, dtype_assign.h:223-371). */
#pragma once
#include "och_dispatch.h"
namespace och {

template <class S, class D, bool SWAP> struct CvtOp
{  typedef S A; typedef D R;
   static OCH_D R f(A x) { if constexpr (SWAP) return cvt<D, S>(byteswap<S>(x)); else return cvt<D, S>(x); }
};

/* one row: fixed source type, all destination types */
template <class S, bool SWAP> struct RowCvt { static const ew2_fn fn[DT_COUNT]; };
#define OCH_X(T) &launch_ew2<CvtOp<S, T, SWAP>>,
template <class S, bool SWAP> const ew2_fn RowCvt<S, SWAP>::fn[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X

#define OCH_COPY_LOOKUP(NAME, T1, T2, T3)                                          \
   ew2_fn copy_lookup_##NAME(int swap, int which, int dst)                         \
   {  if (which == 0) return swap ? RowCvt<T1, true>::fn[dst] : RowCvt<T1, false>::fn[dst]; \
      if (which == 1) return swap ? RowCvt<T2, true>::fn[dst] : RowCvt<T2, false>::fn[dst]; \
      return swap ? RowCvt<T3, true>::fn[dst] : RowCvt<T3, false>::fn[dst];        \
   }
}
