/* TEST INFRASTRUCTURE -- CPU oracle for the MI355X device library.
 *
 * A restatement in plain C (+OpenMP) of the arithmetic and of the threading
 * policy of Ocean's CPU path (Solid CPU kernels, solid/src/core/cpu/ and
 * solid/include/solid/core/{cpu,generic}/). It exists to check the HIP
 * kernels and to time a CPU baseline. Nothing in the product links, loads or
 * calls it; only tests/, the smoke check and the benchmark's cpu_baseline leg
 * may. Operation and type numbering are those of include/ocean_hip.h.
 * All pointers are host pointers; strides are in bytes.
 *
 * What pins each part (tests/test_oracle_ref.py, test_ref_fixtures.py, test_index_cpu.py):
 *   binary / unary operations, conversions (15 x 15, with and without byte swap), half
 *   conversion, reduction step functions: compared with the reference's own macros
 *   (binary_ops.h, unary_ops.h, reduce_ops.h, dtype_assign.h, half.c) compiled from the
 *   reference tree into oracle/_ref/libocean_ref.so; whole operations additionally against
 *   the expected-output files of the reference's example tests (tests/golden/ref/);
 *   index operations: numpy integer-array indexing and the reference's index_008 output; find: numpy.nonzero and the
 *   reference's ocean_find_01 / tensor_find_01 outputs;  integer / bool GEMM: exact arithmetic;
 *   GEMM transposition / conjugation modes for every floating type: the reference's ocean_gemm_02 ... 09d outputs;
 *   reductions (NaN-skipping variants, any / all / nnz along axes, p-norms): ocean_axis_* and ocean_norm_01 / 02 outputs.
 * PARITY UNPINNED (no golden vector, reference build or closed form fixes the bits; the tests
 * hold these to stated tolerances instead):
 *   oracle_gemm for floating and complex types at large sizes -- the reference's CPU result
 *     depends on the BLAS it is linked with; the oracle accumulates in long double and serves
 *     as the exact side of a normwise bound (small integer-valued cases are pinned by
 *     ocean_gemm_01.ref);
 *   transcendental unary functions and floating `power` -- bits depend on the host libm;
 *   the summation order of floating sum / prod / norm over many elements -- thread-count
 *     dependent in the reference; the per-element step functions are pinned, the order is not.
 */
#ifndef ORACLE_H
#define ORACLE_H
#include <stddef.h>
#include <stdint.h>
#include "../include/ocean_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* nthreads: number of OpenMP threads the CPU module would use for one- and
   two-operand loops (<= 1: serial). Three-operand (binary) loops are always serial. */
int oracle_max_threads(void);

int oracle_binary(int op, int dtype, int ndims, const size_t *size,
                  const ptrdiff_t *strides1, void *ptr1, const ptrdiff_t *strides2, void *ptr2,
                  const ptrdiff_t *strides3, void *ptr3);
int oracle_binary_supported(int op, int dtype);
int oracle_unary(int op, int dtype, int ndims, const size_t *size,
                 const ptrdiff_t *strides1, void *ptr1, const ptrdiff_t *strides2, void *ptr2, int nthreads);
int oracle_unary_supported(int op, int dtype);

int oracle_copy(int dtype_src, int dtype_dst,
                int ndims1, const size_t *size1, const ptrdiff_t *strides1, void *ptr1,
                int ndims2, const size_t *size2, const ptrdiff_t *strides2, void *ptr2, int nthreads);
int oracle_byteswap_copy(int dtype_src, int dtype_dst,
                int ndims1, const size_t *size1, const ptrdiff_t *strides1, void *ptr1,
                int ndims2, const size_t *size2, const ptrdiff_t *strides2, void *ptr2, int nthreads);
int oracle_byteswap(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, int nthreads);

int oracle_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                och_scalar value, int nthreads);
int oracle_fill_nan(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                och_scalar value, int nthreads);
int oracle_masked_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides1, void *ptr1,
                const ptrdiff_t *strides2, void *ptr2, och_scalar value, int nthreads);
int oracle_steps_int64(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                int64_t offset, int64_t step, int nthreads);
int oracle_steps_double(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                double offset, double step, int nthreads);
int oracle_steps_cdouble(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                och_cdouble offset, och_cdouble step, int nthreads);

/* Full reductions with the CPU module's threading: per-thread partials over contiguous
   index ranges (threads capped so each gets >= 512 elements), folded in thread order. */
int oracle_reduce_all(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                void *result, int nthreads);
int oracle_reduce_supported(int op, int dtype);
int oracle_reduce_result_dtype(int op, int dtype);
/* Axis reduction; configuration as och_reduce_axis_config (stream ignored). Serial. */
int oracle_reduce_axis(int op, int dtype, const och_reduce_axis_config *config, double p);
/* The same with the outputs split over threads as the CPU module does for many outputs (same bits as the serial form). */
int oracle_reduce_axis_threads(int op, int dtype, const och_reduce_axis_config *config, double p, int nthreads);

/* Column-major GEMM, textbook triple loop; accumulation in the element type. */
int oracle_gemm(int dtype, char transA, char transB, size_t M, size_t N, size_t K,
                const void *alpha, const void *A, ptrdiff_t ldA, const void *B, ptrdiff_t ldB,
                const void *beta, void *C, ptrdiff_t ldC, int nthreads);

/* Index operations (template_index.c): per-dimension offset tables or strides. */
int oracle_add_if_negative(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, och_scalar value);
int oracle_index_to_offset(int dtype, int nstrides, const int64_t *strides, ptrdiff_t stride_reduce, size_t nelem,
                ptrdiff_t stride1, const void *ptr1, ptrdiff_t stride2, void *ptr2);
int oracle_get_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                const ptrdiff_t *strides2, void *ptr2);
int oracle_set_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                const ptrdiff_t *strides2, void *ptr2);
int oracle_fill_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides, void *ptr, och_scalar value);

/* returns the number of non-zero elements; out may be NULL to count only */
size_t oracle_find(int ndims, const size_t *size, const ptrdiff_t *strides, const void *ptr, const int64_t *multiplier, int64_t *out);

/* Software half precision (half.c) exposed for exhaustive tests */
float    oracle_half_to_float(uint16_t h);
uint16_t oracle_float_to_half(float f);

#ifdef __cplusplus
}
#endif
#endif
