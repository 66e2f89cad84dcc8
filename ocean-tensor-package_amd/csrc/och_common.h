/* Shared host-side helpers of the device library: error reporting and the
 * HIP call check. Errors are reported the way Solid does it: functions return
 * -1 and leave a message that the caller can fetch (solid error.h:24-35,
 * imported into Ocean by OC_SOLID_ERRMSG, ocean_solid.h:156-160). */
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/ocean_hip.h"

namespace och {

int  set_error(const char *fmt, ...);        /* stores the message, returns -1 */
void clear_error();
int  gemm_compute_units(void);               /* compute units of the current device (cached per device) */
void note_status(int hip_error);             /* keeps the first error until och_status_check clears it */

/* Every failing runtime call is also noted in a process-wide status that keeps the FIRST error until
   och_status_check reports and clears it (the protocol of src/core/gpu/cuda.c:84-120): work is asynchronous, so the
   call that returns an error is often not the one that caused it, and later calls may fail in its wake. */
#define OCH_CHECK_HIP(CALL)                                                          \
   do { hipError_t _e = (CALL);                                                      \
        if (_e != hipSuccess)                                                        \
        {  och::note_status((int)_e);                                                \
           return och::set_error("%s failed: %s (%s:%d)", #CALL, hipGetErrorString(_e), __FILE__, __LINE__); \
        }                                                                            \
   } while (0)

#define OCH_CHECK_LAUNCH()                                                           \
   do { hipError_t _e = hipGetLastError();                                           \
        if (_e != hipSuccess)                                                        \
        {  och::note_status((int)_e);                                                \
           return och::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(_e), __FILE__, __LINE__); \
        }                                                                            \
   } while (0)

/* After a wait has returned: an error that a kernel or copy raised while it ran shows up as the runtime's last error */
#define OCH_CHECK_AFTER_WAIT(WHAT)                                                   \
   do { hipError_t _e = hipGetLastError();                                           \
        if (_e != hipSuccess)                                                        \
        {  och::note_status((int)_e);                                                \
           return och::set_error("asynchronous error found when %s finished waiting: %s", WHAT, hipGetErrorString(_e)); \
        }                                                                            \
   } while (0)

static inline hipStream_t as_stream(och_stream s) { return (hipStream_t)s; }
/* byte fill by a kernel (och_runtime.hip): unlike a memset node it is safe inside a captured graph */
int fill_bytes(void *dst, int value, size_t nbytes, hipStream_t stream);

/* Scratch memory that kernels of one stream share: work on one stream is ordered, work on different streams is not
   (Ocean gives every storage its own stream), so every (device, stream) pair owns its scratch. It is created on the
   first use of the stream -- or by och_device_warmup / och_stream_begin_capture, so that no allocation happens while
   a stream records -- and released when the stream is destroyed. */
#define OCH_RED_MAX_BLOCKS 512
#define OCH_RED_SLOT 16                               /* bytes per partial of a full reduction */
#define OCH_RED_SCRATCH (OCH_RED_MAX_BLOCKS * OCH_RED_SLOT + 256)
#define OCH_GEMM_WORKSPACE (64u << 20)                /* partial products of the kernels that split K */
struct StreamContext
{  char *red_scratch;          /* OCH_RED_SCRATCH bytes, partial slots + ticket counter (zero between launches) */
   void *host_result;          /* 64 bytes of pinned host memory: result of a full reduction */
   char *gemm_workspace;       /* OCH_GEMM_WORKSPACE bytes, created by stream_gemm_workspace */
};
int stream_context(hipStream_t stream, StreamContext **ctx);
int stream_gemm_workspace(hipStream_t stream, char **workspace);
int stream_release_workspace(hipStream_t stream);
void stream_context_release(hipStream_t stream);
/* device address, on the current device, of the file-scope scratch array of och_reduce_all_device_noalloc (och_reduce.hip) */
int reduce_static_scratch(char **scratch);
#define OCH_RED_NOALLOC_MAX_ELEMENTS (1ull << 40)

} /* namespace och */
