/* Row of launchers (one per element type) for a unary operation id. */
#pragma once
#include "och_dispatch.h"
#include "och_ops_unary.h"
namespace och {
template <int ID> struct RowU { static const ew2_fn fn[DT_COUNT]; };
#define OCH_X(T) Pick2<UnaryOp<T, ID>, unary_defined<T, ID>()>::fn,
template <int ID> const ew2_fn RowU<ID>::fn[DT_COUNT] = { OCH_FOR_ALL_TYPES(OCH_X) };
#undef OCH_X
}
