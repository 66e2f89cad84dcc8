/* C ABI of the full reductions (och_reduce_all and its queries). Without a caller's buffer they use the scratch of
 * the stream they run on. */
#include "och_reduce_all.h"
#include <string.h>
#include <atomic>
#include <mutex>

namespace och {
/* the instantiations are spread over eight translation units (build time); each knows its own operations */
#define OCH_RED_PARTS(X) X(a) X(b) X(c) X(d) X(e) X(f) X(g) X(h)
#define OCH_X(part) red_fn reduce_lookup_##part(int op, int dtype);
OCH_RED_PARTS(OCH_X)
#undef OCH_X
static_assert((int)R_COUNT == (int)OCH_REDUCE_COUNT && (int)R_NORM2_NAN == (int)OCH_R_NORM2_NAN && (int)R_SUM == (int)OCH_R_SUM,
              "operation lists out of step");

static red_fn reduce_lookup(int op, int dtype)
{
   if (dtype < 0 || dtype >= DT_COUNT || op < 0 || op >= OCH_REDUCE_COUNT) return nullptr;
   red_fn fn = nullptr;
#define OCH_X(part) if (fn == nullptr) fn = reduce_lookup_##part(op, dtype);
   OCH_RED_PARTS(OCH_X)
#undef OCH_X
   return fn;
}

}  /* namespace och */

using namespace och;

extern "C" size_t och_reduce_all_buffer_size(void) { return OCH_RED_SCRATCH; }
extern "C" int och_reduce_supported(int op, int dtype) { return reduce_lookup(op, dtype) != nullptr; }

extern "C" int och_reduce_result_dtype(int op, int dtype)
{
   if (!och_reduce_supported(op, dtype)) return -1;
   const bool isbool = dtype == OCH_BOOL, isuint = dtype >= OCH_UINT8 && dtype <= OCH_UINT64;
   const bool issint = dtype >= OCH_INT8 && dtype <= OCH_INT64, iscomplex = dtype >= OCH_CHALF;
   const int abstype = iscomplex ? dtype - 3 : (issint ? dtype - 4 : dtype);
   if (op <= OCH_R_ANY_NAN || (op >= OCH_R_ALL_LT && op <= OCH_R_ALL_GELE)) return OCH_BOOL;
   if (op == OCH_R_NNZ || op == OCH_R_NNZ_NAN) return OCH_UINT64;
   if (op >= OCH_R_SUM && op <= OCH_R_PROD_NAN) return (isbool || isuint) ? OCH_UINT64 : (issint ? OCH_INT64 : dtype);
   if (op == OCH_R_SUM_ABS || op == OCH_R_SUM_ABS_NAN) return (isbool || isuint || issint) ? OCH_UINT64 : abstype;
   if (op == OCH_R_MAXIMUM || op == OCH_R_MINIMUM) return dtype;
   if (op == OCH_R_MAXIMUM_ABS || op == OCH_R_MINIMUM_ABS) return abstype;
   return (isbool || isuint || issint) ? OCH_DOUBLE : abstype;      /* norms */
}

namespace och {
static std::atomic<uint64_t> g_part_limit(OCH_RED_PART_LIMIT);
uint64_t reduce_part_limit() { return g_part_limit.load(); }
}
extern "C" void och_reduce_set_part_limit(size_t nelem)
{  och::g_part_limit.store((nelem == 0 || nelem > OCH_RED_PART_LIMIT) ? OCH_RED_PART_LIMIT : (uint64_t)nelem); }
extern "C" long long och_reduce_cut_parts(int ndims, const size_t *size, size_t limit, long long max_boxes, size_t *starts, size_t *counts)
{
   if (ndims < 1 || ndims > OCH_MAX_DIMS) return -1;
   uint64_t sz[OCH_MAX_DIMS]; long long kept = 0;
   for (int d = 0; d < ndims; d++) sz[d] = size[d];
   return (long long)och::reduce_cut_parts(ndims, sz, (uint64_t)limit, [&](const uint64_t *start, const uint64_t *count)
          {  if (kept < max_boxes)
             {  for (int d = 0; d < ndims; d++) { starts[kept * ndims + d] = start[d]; counts[kept * ndims + d] = count[d]; }
                kept++;
             }
          });
}

extern "C" int och_reduce_all_device(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                   void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                   void *dresult, void *buffer, och_stream stream)
{
   red_fn fn = reduce_lookup(op, dtype);
   if (fn == nullptr) return set_error("reduction %d is not available for data type %d", op, dtype);
   char *scratch = (char *)buffer;
   if (scratch == nullptr)
   {  StreamContext *ctx;
      if (stream_context(as_stream(stream), &ctx) != 0) return -1;
      scratch = ctx->red_scratch;
   }
   return fn(ndims, size, strides, ptr, param1, param2, p, dresult, scratch, buffer != nullptr, as_stream(stream));
}

/* ---- the entry point that allocates nothing ------------------------------------------------
   Same kernels as och_reduce_all_device; the partial slots and the ticket counter live in a
   file-scope device array instead of memory that the library or the caller allocates. The array's
   name is only a host-side handle: its device address is asked for once per device (each device
   holds its own copy at its own address) and only that address is ever handed to a kernel. */
#define OCH_RED_STATIC_DEVICES 64
static __device__ __align__(256) unsigned char scratch[OCH_RED_SCRATCH];
static char *g_static_scratch[OCH_RED_STATIC_DEVICES];
static std::mutex g_static_scratch_mutex;

namespace och {
int reduce_static_scratch(char **out)
{
   int dev;
   OCH_CHECK_HIP(hipGetDevice(&dev));
   if (dev < 0 || dev >= OCH_RED_STATIC_DEVICES) return set_error("device index %d is beyond the %d devices the static scratch covers", dev, OCH_RED_STATIC_DEVICES);
   std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
   if (g_static_scratch[dev] == nullptr)
   {  void *ptr = nullptr;
      OCH_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
      if (ptr == nullptr) return set_error("the static reduction scratch has no address on device %d", dev);
      g_static_scratch[dev] = (char *)ptr;
   }
   *out = g_static_scratch[dev];
   return 0;
}
}

extern "C" size_t och_reduce_all_noalloc_max_elements(void) { return (size_t)OCH_RED_NOALLOC_MAX_ELEMENTS; }

extern "C" int och_reduce_all_device_noalloc(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                   void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                   void *dresult, och_stream stream)
{
   red_fn fn = reduce_lookup(op, dtype);
   if (fn == nullptr) return set_error("reduction %d is not available for data type %d", op, dtype);
   if (ndims < 0 || ndims > OCH_MAX_DIMS) return set_error("invalid number of dimensions (%d)", ndims);
   if (dresult == nullptr) return set_error("och_reduce_all_device_noalloc: null result pointer");
   unsigned long long nelem = 1;
   for (int d = 0; d < ndims; d++)
   {  if (size[d] != 0 && nelem > OCH_RED_NOALLOC_MAX_ELEMENTS / size[d])
         return set_error("och_reduce_all_device_noalloc: more than %llu elements; use och_reduce_all_device", (unsigned long long)OCH_RED_NOALLOC_MAX_ELEMENTS);
      nelem *= size[d];
   }
   char *dscratch;
   if (reduce_static_scratch(&dscratch) != 0) return -1;
   /* the array keeps what the last call (or a failed launch) left: the counter is cleared by a small fill kernel on
      this stream in front of every reduction; the partial slots need no clearing (every slot that is read was written
      by this launch) */
   return fn(ndims, size, strides, ptr, param1, param2, p, dresult, dscratch, true, as_stream(stream));
}

extern "C" int och_reduce_all(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                   void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                   void *result, void *buffer, och_stream stream)
{
   StreamContext *ctx;
   if (stream_context(as_stream(stream), &ctx) != 0) return -1;
   /* the kernel writes the scalar straight into pinned host memory; one synchronisation */
   if (och_reduce_all_device(op, dtype, ndims, size, strides, ptr, param1, param2, p, ctx->host_result, buffer, stream) != 0) return -1;
   OCH_CHECK_HIP(hipStreamSynchronize(as_stream(stream)));
   int rd = och_reduce_result_dtype(op, dtype);
   memcpy(result, ctx->host_result, och_type_size[rd]);
   return 0;
}
