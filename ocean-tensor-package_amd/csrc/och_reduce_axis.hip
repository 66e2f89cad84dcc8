/* C ABI of the axis reductions (och_reduce_axis). The 21 operations of the reference's axis
 * family (solid_core_gpu.src: axis_any ... axis_norm2_nan) are available; the range checks
 * (all_lt ...) exist as full reductions only. */
#include "och_reduce_axis.h"
#include <atomic>
namespace och {
static std::atomic<uint64_t> g_axis_output_limit(0xFFFFFF00ull);
uint64_t axis_output_limit() { return g_axis_output_limit.load(); }
static std::atomic<uint64_t> g_axis_range_limit(0xFFFFFF00ull);
uint64_t axis_range_limit() { return g_axis_range_limit.load(); }
/* the instantiations are spread over eight translation units (build time); each knows its own operations */
#define OCH_AXIS_PARTS(X) X(a) X(b) X(c) X(d) X(e) X(f) X(g) X(h)
#define OCH_X(part) axis_fn axis_lookup_##part(int op, int dtype);
OCH_AXIS_PARTS(OCH_X)
#undef OCH_X
}
extern "C" void och_reduce_axis_set_output_limit(size_t outputs)
{  och::g_axis_output_limit.store((outputs == 0 || outputs > 0xFFFFFF00ull) ? 0xFFFFFF00ull : (uint64_t)outputs); }
extern "C" void och_reduce_axis_set_range_limit(size_t nelem)
{  och::g_axis_range_limit.store((nelem == 0 || nelem > 0xFFFFFF00ull) ? 0xFFFFFF00ull : (uint64_t)nelem); }
extern "C" int och_reduce_axis(int op, int dtype, const och_reduce_axis_config *config, double p)
{
   using namespace och;
   axis_fn fn = nullptr;
   if (dtype >= 0 && dtype < DT_COUNT)
   {
#define OCH_X(part) if (fn == nullptr) fn = axis_lookup_##part(op, dtype);
      OCH_AXIS_PARTS(OCH_X)
#undef OCH_X
   }
   if (fn == nullptr) return set_error("axis reduction %d is not available for data type %d", op, dtype);
   return fn(config, p);
}
