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

#define OCH_CHECK_HIP(CALL)                                                          \
   do { hipError_t _e = (CALL);                                                      \
        if (_e != hipSuccess)                                                        \
           return och::set_error("%s failed: %s (%s:%d)", #CALL, hipGetErrorString(_e), __FILE__, __LINE__); \
   } while (0)

#define OCH_CHECK_LAUNCH()                                                           \
   do { hipError_t _e = hipGetLastError();                                           \
        if (_e != hipSuccess)                                                        \
           return och::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(_e), __FILE__, __LINE__); \
   } while (0)

static inline hipStream_t as_stream(och_stream s) { return (hipStream_t)s; }
/* byte fill by a kernel (och_runtime.hip): unlike a memset node it is safe inside a captured graph */
int fill_bytes(void *dst, int value, size_t nbytes, hipStream_t stream);
/* creates the current device's reduction scratch and pinned result slot if they do not exist yet (och_reduce.hip) */
int red_context_init();

} /* namespace och */
