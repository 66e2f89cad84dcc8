/* Host build of csrc/och_math.h beside the host's libm, for tests/test_math_cpu.py: the routines use IEEE basic operations
   only, so what this file computes on the CPU is what the kernels compute on the device. */
#include <math.h>
#include <stddef.h>
#include "och_math.h"

extern "C" void host_och_powf(size_t n, const float *x, const float *y, float *out) { for (size_t i = 0; i < n; i++) out[i] = och::och_powf(x[i], y[i]); }
extern "C" void host_libm_powf(size_t n, const float *x, const float *y, float *out) { for (size_t i = 0; i < n; i++) out[i] = powf(x[i], y[i]); }
extern "C" void host_och_tanh(size_t n, const double *x, double *out) { for (size_t i = 0; i < n; i++) out[i] = och::och_tanh(x[i]); }
extern "C" void host_libm_tanh(size_t n, const double *x, double *out) { for (size_t i = 0; i < n; i++) out[i] = tanh(x[i]); }
