/* TEST INFRASTRUCTURE (see oracle.h).
 * Column-major GEMM C <- alpha * op(A) * op(B) + beta * C as a textbook triple loop.
 * Semantics of the call follow src/core/cpu/op/tensor_blas_cpu.c:61-178 (M or N zero: no-op;
 * K zero: C <- beta*C) and, for bool / integers, solid/src/core/cpu/template_blas.c
 * (bool: + is OR, * is AND; integers wrap). Floating and complex types accumulate each dot
 * product in long double, so that the result can serve as the "exact" side of a normwise
 * error bound; Ocean's own CPU result depends on whichever BLAS it was linked with and is
 * not pinned by the reference (its vendored fallback even mis-scales C for beta outside
 * {0,1}, src/external/ocean-blas/ocean_custom_blas.c:101,126).
 */
#include "oracle.h"
#include "oracle_convert.h"
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define IDX(P, ld, i, j, tr) ((tr) ? (P)[(size_t)(j) + (size_t)(i) * (ld)] : (P)[(size_t)(i) + (size_t)(j) * (ld)])

#define GEMM_REAL(NAME, T, ACC, LOAD, STORE)                                                  \
static void NAME(int ta, int tb, size_t M, size_t N, size_t K, const void *alpha, const void *A, ptrdiff_t ldA, \
                 const void *B, ptrdiff_t ldB, const void *beta, void *C, ptrdiff_t ldC, int nthreads) \
{  const T *a = (const T *)A, *b = (const T *)B; T *c = (T *)C;                               \
   ACC al = LOAD(*(const T *)alpha), be = LOAD(*(const T *)beta);                             \
   ptrdiff_t j;                                                                               \
   _Pragma("omp parallel for num_threads(nthreads) schedule(static)")                         \
   for (j = 0; j < (ptrdiff_t)N; j++)                                                         \
   {  size_t i, k;                                                                            \
      for (i = 0; i < M; i++)                                                                 \
      {  ACC s = 0;                                                                           \
         for (k = 0; k < K; k++) s += (ACC)LOAD(IDX(a, ldA, i, k, ta)) * (ACC)LOAD(IDX(b, ldB, k, j, tb)); \
         { ACC r = al * s; if (be != 0) r += be * (ACC)LOAD(c[i + (size_t)j * ldC]); c[i + (size_t)j * ldC] = STORE(r); } \
      }                                                                                       \
   }                                                                                          \
}
#define ID(x) (x)
#define H2F(x) o_half_to_float(x)
#define F2H(x) o_float_to_half((float)(x))
GEMM_REAL(o_gemm_float, float, long double, ID, (float))
GEMM_REAL(o_gemm_double, double, long double, ID, (double))
GEMM_REAL(o_gemm_half, o_half, double, H2F, F2H)

/* integers: wrap-around arithmetic in the unsigned twin */
#define GEMM_INT(NAME, T, UT)                                                                 \
static void NAME(int ta, int tb, size_t M, size_t N, size_t K, const void *alpha, const void *A, ptrdiff_t ldA, \
                 const void *B, ptrdiff_t ldB, const void *beta, void *C, ptrdiff_t ldC, int nthreads) \
{  const T *a = (const T *)A, *b = (const T *)B; T *c = (T *)C;                               \
   UT al = (UT)*(const T *)alpha, be = (UT)*(const T *)beta; size_t i, j, k; (void)nthreads;  \
   for (j = 0; j < N; j++) for (i = 0; i < M; i++)                                            \
   {  UT s = 0;                                                                               \
      for (k = 0; k < K; k++) s = (UT)(s + (UT)((UT)IDX(a, ldA, i, k, ta) * (UT)IDX(b, ldB, k, j, tb))); \
      s = (UT)(al * s);                                                                       \
      if (be != 0) s = (UT)(s + (UT)(be * (UT)c[i + j * ldC]));                               \
      c[i + j * ldC] = (T)s;                                                                  \
   }                                                                                          \
}
GEMM_INT(o_gemm_uint8, uint8_t, uint8_t)   GEMM_INT(o_gemm_uint16, uint16_t, uint16_t)
GEMM_INT(o_gemm_uint32, uint32_t, uint32_t) GEMM_INT(o_gemm_uint64, uint64_t, uint64_t)
GEMM_INT(o_gemm_int8, int8_t, uint8_t)     GEMM_INT(o_gemm_int16, int16_t, uint16_t)
GEMM_INT(o_gemm_int32, int32_t, uint32_t)  GEMM_INT(o_gemm_int64, int64_t, uint64_t)

static void o_gemm_bool(int ta, int tb, size_t M, size_t N, size_t K, const void *alpha, const void *A, ptrdiff_t ldA,
                 const void *B, ptrdiff_t ldB, const void *beta, void *C, ptrdiff_t ldC, int nthreads)
{  const o_bool *a = (const o_bool *)A, *b = (const o_bool *)B; o_bool *c = (o_bool *)C;
   o_bool al = *(const o_bool *)alpha, be = *(const o_bool *)beta; size_t i, j, k; (void)nthreads;
   for (j = 0; j < N; j++) for (i = 0; i < M; i++)
   {  o_bool s = 0;
      for (k = 0; k < K; k++) s |= (o_bool)(IDX(a, ldA, i, k, ta) & IDX(b, ldB, k, j, tb));
      s &= al;
      if (be) s |= c[i + j * ldC];
      c[i + j * ldC] = s ? 1 : 0;
   }
}

/* complex: trans 'C' conjugates */
#define GEMM_CPLX(NAME, T, PT, LOAD, STORE)                                                   \
static void NAME(int ta, int tb, size_t M, size_t N, size_t K, const void *alpha, const void *A, ptrdiff_t ldA, \
                 const void *B, ptrdiff_t ldB, const void *beta, void *C, ptrdiff_t ldC, int nthreads) \
{  const T *a = (const T *)A, *b = (const T *)B; T *c = (T *)C;                               \
   long double alr = LOAD(((const T *)alpha)->real), ali = LOAD(((const T *)alpha)->imag);    \
   long double ber = LOAD(((const T *)beta)->real), bei = LOAD(((const T *)beta)->imag);      \
   int tra = (ta != 0), trb = (tb != 0); long double sa = (ta == 2) ? -1 : 1, sb = (tb == 2) ? -1 : 1; \
   ptrdiff_t j;                                                                               \
   _Pragma("omp parallel for num_threads(nthreads) schedule(static)")                         \
   for (j = 0; j < (ptrdiff_t)N; j++)                                                         \
   {  size_t i, k;                                                                            \
      for (i = 0; i < M; i++)                                                                 \
      {  long double sr = 0, si = 0, rr, ri;                                                  \
         for (k = 0; k < K; k++)                                                              \
         {  T x = IDX(a, ldA, i, k, tra), y = IDX(b, ldB, k, j, trb);                         \
            long double xr = LOAD(x.real), xi = sa * LOAD(x.imag), yr = LOAD(y.real), yi = sb * LOAD(y.imag); \
            sr += xr * yr - xi * yi; si += xr * yi + xi * yr;                                 \
         }                                                                                    \
         rr = alr * sr - ali * si; ri = alr * si + ali * sr;                                  \
         if (ber != 0 || bei != 0)                                                            \
         {  long double cr = LOAD(c[i + (size_t)j * ldC].real), ci = LOAD(c[i + (size_t)j * ldC].imag); \
            rr += ber * cr - bei * ci; ri += ber * ci + bei * cr;                             \
         }                                                                                    \
         c[i + (size_t)j * ldC].real = STORE(rr); c[i + (size_t)j * ldC].imag = STORE(ri);    \
      }                                                                                       \
   }                                                                                          \
}
GEMM_CPLX(o_gemm_cfloat, o_cfloat, float, ID, (float))
GEMM_CPLX(o_gemm_cdouble, o_cdouble, double, ID, (double))
GEMM_CPLX(o_gemm_chalf, o_chalf, o_half, H2F, F2H)

typedef void (*o_gemm_fn)(int, int, size_t, size_t, size_t, const void *, const void *, ptrdiff_t, const void *, ptrdiff_t,
                          const void *, void *, ptrdiff_t, int);
static const o_gemm_fn o_gemm_table[O_NTYPES] = {
   o_gemm_bool, o_gemm_uint8, o_gemm_uint16, o_gemm_uint32, o_gemm_uint64, o_gemm_int8, o_gemm_int16, o_gemm_int32, o_gemm_int64,
   o_gemm_half, o_gemm_float, o_gemm_double, o_gemm_chalf, o_gemm_cfloat, o_gemm_cdouble };

static int o_trans(char t) { return (t == 'N' || t == 'n') ? 0 : ((t == 'T' || t == 't') ? 1 : ((t == 'C' || t == 'c') ? 2 : -1)); }

int oracle_gemm(int dtype, char transA, char transB, size_t M, size_t N, size_t K,
                const void *alpha, const void *A, ptrdiff_t ldA, const void *B, ptrdiff_t ldB,
                const void *beta, void *C, ptrdiff_t ldC, int nthreads)
{
   int ta = o_trans(transA), tb = o_trans(transB);
   if (dtype < 0 || dtype >= O_NTYPES || ta < 0 || tb < 0) return -1;
   if (M == 0 || N == 0) return 0;
   if (nthreads < 1) nthreads = 1;
   if (dtype < O_CHALF) { ta = (ta != 0); tb = (tb != 0); }      /* conjugation of a real value is the identity */
   o_gemm_table[dtype](ta, tb, M, N, K, alpha, A, ldA, B, ldB, beta, C, ldC, nthreads);
   return 0;
}
