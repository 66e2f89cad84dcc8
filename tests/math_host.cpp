/* Host build of csrc/och_math.h beside the host's libm, for tests/test_math_cpu.py: the routines use IEEE basic operations
   only, so what this file computes on the CPU is what the kernels compute on the device. */
#include <math.h>
#include <stddef.h>
#include "och_math.h"

extern "C" void host_och_powf(size_t n, const float *x, const float *y, float *out) { for (size_t i = 0; i < n; i++) out[i] = och::och_powf(x[i], y[i]); }
extern "C" void host_libm_powf(size_t n, const float *x, const float *y, float *out) { for (size_t i = 0; i < n; i++) out[i] = powf(x[i], y[i]); }
extern "C" void host_och_tanh(size_t n, const double *x, double *out) { for (size_t i = 0; i < n; i++) out[i] = och::och_tanh(x[i]); }
extern "C" void host_libm_tanh(size_t n, const double *x, double *out) { for (size_t i = 0; i < n; i++) out[i] = tanh(x[i]); }

#define ONE(NAME, T, MINE, LIBM) \
   extern "C" void host_och_##NAME(size_t n, const T *x, T *out) { for (size_t i = 0; i < n; i++) out[i] = och::MINE(x[i]); } \
   extern "C" void host_libm_##NAME(size_t n, const T *x, T *out) { for (size_t i = 0; i < n; i++) out[i] = LIBM(x[i]); }
ONE(sinh, double, och_sinh, sinh)   ONE(cosh, double, och_cosh, cosh)
ONE(sinhf, float, och_sinhf, sinhf) ONE(coshf, float, och_coshf, coshf)
ONE(log1p, double, och_log1p, log1p)   ONE(atanh, double, och_atanh, atanh)   ONE(asinh, double, och_asinh, asinh)   ONE(acosh, double, och_acosh, acosh)
ONE(log1pf, float, och_log1pf, log1pf) ONE(atanhf, float, och_atanhf, atanhf) ONE(asinhf, float, och_asinhf, asinhf) ONE(acoshf, float, och_acoshf, acoshf)
