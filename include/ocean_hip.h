/* ------------------------------------------------------------------------ */
/* ocean_hip.h -- C ABI of the MI355X (gfx950) device library for Ocean's   */
/* core module.                                                             */
/*                                                                          */
/* Every entry point is plain C: pointers, sizes, byte strides and an       */
/* opaque stream handle (a hipStream_t). The library replaces the Solid GPU */
/* foundation (solid_gpu_<op>_<type> / solid_gpu_<op>[dtype] tables,        */
/* solid/src/core/gpu/solid_core_gpu.src:42-439) and the CUDA runtime and   */
/* cuBLAS calls made by Ocean's GPU device module (files in src/core/gpu). The */
/* reference exports one symbol per (operation, type); this library takes   */
/* the operation and the element type as leading integer arguments, so that */
/* a lookup `solid_gpu_add[dtype](...)` becomes `och_binary(OCH_ADD, dtype, */
/* ...)` with the remaining arguments unchanged.                            */
/*                                                                          */
/* Conventions (same as Solid, solid_core_gpu.src:20-28):                   */
/*   - sizes are element counts, strides are in BYTES and may be zero       */
/*     (broadcast) or, for source operands, negative;                       */
/*   - at most OCH_MAX_DIMS dimensions;                                     */
/*   - all device pointers belong to the current HIP device;                */
/*   - functions return 0 on success and -1 on error; och_last_error()      */
/*     returns the message (cf. solid_errmsg, solid error.h:24-35).         */
/* All launches are asynchronous on the given stream unless stated.         */
/* ------------------------------------------------------------------------ */
#ifndef OCEAN_HIP_H
#define OCEAN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OCH_MAX_DIMS 8

/* Element types; numbering identical to OcDType (include/ocean/base/dtype.h:29-36)
   and to Solid's type index (solid/include/solid/base/generic/dtype_macros.h:133-147). */
typedef enum {
   OCH_BOOL = 0, OCH_UINT8, OCH_UINT16, OCH_UINT32, OCH_UINT64,
   OCH_INT8, OCH_INT16, OCH_INT32, OCH_INT64,
   OCH_HALF, OCH_FLOAT, OCH_DOUBLE,
   OCH_CHALF, OCH_CFLOAT, OCH_CDOUBLE,
   OCH_DTYPE_COUNT
} och_dtype;

/* Scalar passed by value; mirrors solid_scalar (solid/include/solid/base/generic/scalar.h:30-50). */
typedef struct { uint16_t real, imag; } och_chalf;
typedef struct { float    real, imag; } och_cfloat;
typedef struct { double   real, imag; } och_cdouble;
typedef union {
   uint8_t  _bool;  uint8_t  _uint8; uint16_t _uint16; uint32_t _uint32; uint64_t _uint64;
   int8_t   _int8;  int16_t  _int16; int32_t  _int32;  int64_t  _int64;
   uint16_t _half;  float    _float; double   _double;
   och_chalf _chalf; och_cfloat _cfloat; och_cdouble _cdouble;
} och_scalar;

typedef void *och_stream;   /* hipStream_t */
typedef void *och_event;    /* hipEvent_t  */

/* Element size in bytes per dtype (solid_gpu_type_size[], solid_core_gpu.src:34). */
extern const int och_type_size[OCH_DTYPE_COUNT];

/* Message of the most recent failure in the calling thread. */
const char *och_last_error(void);

/* The first runtime error since the last check (OcCuda_setStatus / OcCuda_checkStatus / OcCuda_clearStatus,            */
/* src/core/gpu/cuda.c:84-120). Work is asynchronous: an error raised by a kernel or a copy while it runs is seen by   */
/* whichever call looks next, and calls after it may fail in its wake. Every failing call of this library notes its    */
/* error code; the first one is kept. och_stream_synchronize, och_event_synchronize and och_device_synchronize also    */
/* ask the runtime, once the wait is over, for an error raised meanwhile, note it and return -1 with a message that    */
/* says where it was found. och_status_check returns 0 when nothing was noted; otherwise -1 with "HIP error: ..." as   */
/* the message, and forgets the error. och_status_clear forgets it without reporting.                                  */
int  och_status_check(void);
void och_status_clear(void);

/* ======================================================================== */
/* Device, stream, event and memory glue                                    */
/* Replaces: src/core/gpu/device_gpu.c:155-420 (warm-up, streams, events),  */
/*           src/core/gpu/storage_gpu.c:61-302 (alloc/free/copy/zero),      */
/*           src/core/gpu/cuda.c:67-120 (set device, sticky status),        */
/*           solid/src/base/gpu/solid_gpu.c:28-236 (property cache).        */
/* ======================================================================== */
typedef struct {
   char     name[256];
   char     arch[64];                 /* e.g. "gfx950:sramecc+:xnack-" */
   size_t   total_global_mem;
   size_t   shared_mem_per_block;     /* LDS bytes per workgroup */
   int      multiprocessor_count;     /* compute units */
   int      wavefront_size;
   int      max_threads_per_block;
   int      max_threads_per_multiprocessor;
   int      clock_rate_khz;
   int      memory_clock_rate_khz;
   int      memory_bus_width;
   int      l2_cache_size;
   int      pci_bus_id, pci_device_id, pci_domain_id;
   int      concurrent_kernels;
   int      ecc_enabled;
   /* the remaining fields of OcDevicePropGPU (include/ocean/core/gpu/device_gpu.h:31-75) that HIP reports */
   size_t   free_global_mem;          /* at the time of the query; och_device_mem_info refreshes it */
   size_t   total_const_mem;
   size_t   mem_pitch;
   int      regs_per_block;
   int      max_threads_dim[3];
   int      max_grid_size[3];
   int      major, minor;             /* gfx950 reports 9.5 */
   int      async_engine_count;       /* > 0: copies overlap kernels (deviceOverlap) */
   int      kernel_exec_timeout_enabled;
   int      integrated;
   int      can_map_host_memory;
   int      compute_mode;
   int      tcc_driver;               /* always 0 */
} och_device_prop;

int och_device_count(int *count);                          /* device_gpu.c:184 cudaGetDeviceCount */
int och_device_set(int device);                            /* cuda.c:67 OcCuda_setDevice */
int och_device_get(int *device);
int och_device_properties(int device, och_device_prop *p); /* device_gpu.c:471-616 */
int och_device_mem_info(int device, size_t *free_bytes, size_t *total_bytes); /* device_gpu.c:620-637 updateProperties */
int och_device_can_access_peer(int device, int peer, int *result); /* device_gpu.c:447-454 */
int och_device_warmup(int device);                         /* device_gpu.c:155-172 + template_dummy.cu:21-37 */
int och_device_synchronize(void);

int och_stream_create(och_stream *stream);                 /* device_gpu.c:251-288 */
int och_stream_destroy(och_stream stream);                 /* device_gpu.c:324-346 */
int och_stream_synchronize(och_stream stream);             /* device_gpu.c:374-382 */
/* No counterpart in the reference. Products that are cut along K, matrix-vector products and sliced axis reductions  */
/* keep partial results in a 64 MB workspace that belongs to the stream (taken from the stream-ordered pool at the     */
/* first such call, or by och_stream_begin_capture; released with the stream). A caller that retires a stream without */
/* destroying it -- Ocean's device layer recycles up to 64 of them -- gives the workspace back with this call; it is   */
/* freed behind the work already queued on the stream and the next call that needs one takes a new one. A graph         */
/* recorded on the stream addresses the old workspace and must not be launched after this call.                        */
int och_stream_release_workspace(och_stream stream);
int och_stream_wait_event(och_stream stream, och_event event); /* device_gpu.c:411-420 */
int och_event_create(och_event *event, int timing);        /* device_gpu.c:292-320; timing=0: disable timing */
int och_event_destroy(och_event event);                    /* device_gpu.c:350-370 */
int och_event_record(och_event event, och_stream stream);  /* device_gpu.c:398-407 */
int och_event_synchronize(och_event event);                /* device_gpu.c:386-394 */
int och_event_elapsed_ms(och_event start, och_event stop, float *ms);

/* Launch-bound sequences of small operations (the dot -> scale -> subtract chain of a modified Gram-Schmidt sweep   */
/* issues millions of them) can be recorded once and replayed as one graph launch. No counterpart in the reference  */
/* (it launches every operation separately). Between begin and end the stream records instead of executing; calls   */
/* that synchronise or allocate may not be recorded: och_reduce_all, och_find_count, och_memcpy_htod / dtoh,        */
/* och_malloc_async / och_free_async, och_copy between tensors of different shape AND type. Everything else in this */
/* header is recordable; scalars passed in host memory are frozen at their recorded value, scalars in device memory */
/* are read at every replay. `stream` must be a created stream. A graph replays on the stream that recorded it and on */
/* no other (och_graph_launch returns an error): its reductions and split products use that stream's scratch memory,  */
/* which a replay elsewhere would share, unordered, with the work of the recording stream.                           */
typedef void *och_graph;
int och_stream_begin_capture(och_stream stream);
int och_stream_end_capture(och_stream stream, och_graph *graph);
int och_graph_launch(och_graph graph, och_stream stream);
int och_graph_destroy(och_graph graph);

/* Stream-ordered allocation: the block is usable by work enqueued on `stream`
   after the call and is returned to the device pool in stream order.
   Replaces cudaMalloc/cudaFree of storage_gpu.c:83-95,107-116. */
int och_malloc_async(void **ptr, size_t nbytes, och_stream stream);
int och_free_async(void *ptr, och_stream stream);
int och_malloc_host(void **ptr, size_t nbytes);            /* pinned host memory */
int och_free_host(void *ptr);
int och_memcpy_dtod_async(void *dst, const void *src, size_t nbytes, och_stream stream); /* storage_gpu.c:120-161 */
int och_memcpy_peer_async(void *dst, int dst_device, const void *src, int src_device, size_t nbytes, och_stream stream);
int och_memcpy_htod(void *dst, const void *src, size_t nbytes, och_stream stream);  /* storage_gpu.c:165-189; returns after completion */
int och_memcpy_dtoh(void *dst, const void *src, size_t nbytes, och_stream stream);  /* storage_gpu.c:194-221; returns after completion */
int och_memcpy_htod_async(void *dst, const void *src, size_t nbytes, och_stream stream);
int och_memcpy_dtoh_async(void *dst, const void *src, size_t nbytes, och_stream stream);
int och_memset_async(void *dst, int value, size_t nbytes, och_stream stream);       /* storage_gpu.c:283-302 */

/* ======================================================================== */
/* Fill, steps (elemwise1)                                                  */
/* Replaces solid_gpu_fill / fill_nan / masked_fill (template_fill.cu:35-82)*/
/* and steps_int64/double/cdouble (template_steps.cu:31-57).                */
/* fill_nan follows the CPU semantics (only NaN entries are replaced,       */
/* unary_ops.h:332-334,669-672); the reference GPU kernel overwrote all.    */
/* ======================================================================== */
int och_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
             void *ptr, och_scalar value, och_stream stream);
int och_fill_nan(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                 void *ptr, och_scalar value, och_stream stream);
/* ptr1: data (dtype), ptr2: mask (bool) */
int och_masked_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides1,
                    void *ptr1, const ptrdiff_t *strides2, void *ptr2,
                    och_scalar value, och_stream stream);
int och_steps_int64(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                    void *ptr, int64_t offset, int64_t step, och_stream stream);
int och_steps_double(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                     void *ptr, double offset, double step, och_stream stream);
int och_steps_cdouble(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                      void *ptr, och_cdouble offset, och_cdouble step, och_stream stream);

/* ======================================================================== */
/* Copy with type conversion, byteswap                                      */
/* och_copy replaces solid_gpu_copy[src][dst] (template_copy.cu:55-86):     */
/*   operand 1 is the source, operand 2 the destination; the shapes may     */
/*   differ as long as the element counts match (reshape copy).             */
/* och_byteswap / och_byteswap_copy have no GPU counterpart in the          */
/*   reference; they replace solid_cpu_byteswap (template_byteswap.c:27-34) */
/*   and solid_cpu_byteswap_copy (template_copy.c:79-89): each real part is */
/*   byte-reversed; byteswap_copy reverses the SOURCE element first and     */
/*   then converts (dtype_assign.h:297-371).                                */
/* ======================================================================== */
int och_copy(int dtype_src, int dtype_dst,
             int ndims1, const size_t *size1, const ptrdiff_t *strides1, void *ptr1,
             int ndims2, const size_t *size2, const ptrdiff_t *strides2, void *ptr2,
             och_stream stream);
int och_byteswap_copy(int dtype_src, int dtype_dst,
             int ndims1, const size_t *size1, const ptrdiff_t *strides1, void *ptr1,
             int ndims2, const size_t *size2, const ptrdiff_t *strides2, void *ptr2,
             och_stream stream);
int och_byteswap(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                 void *ptr, och_stream stream);

/* ======================================================================== */
/* Unary elementwise: y = f(x)  (template_unary.cu:52-244)                  */
/* Order follows include/ocean/core/generic/generate_tensor_unary.h:19-62.  */
/* ptr2/strides2 NULL selects the in-place form. Output type: same as the   */
/* input except OCH_ABSOLUTE on complex (real part type) and OCH_IS* (bool).*/
/* ======================================================================== */
typedef enum {
   OCH_NEGATIVE = 0, OCH_BITWISE_NOT, OCH_LOGICAL_NOT, OCH_CONJ, OCH_RECIPROCAL,
   OCH_SIN, OCH_COS, OCH_TAN, OCH_SINH, OCH_COSH, OCH_TANH,
   OCH_ARCSIN, OCH_ARCCOS, OCH_ARCTAN, OCH_ARCSINH, OCH_ARCCOSH, OCH_ARCTANH,
   OCH_SQRT, OCH_CBRT, OCH_SQUARE, OCH_EXP, OCH_EXP2, OCH_EXP10, OCH_EXPM1,
   OCH_LOG, OCH_LOG2, OCH_LOG10, OCH_LOG1P,
   OCH_ABSOLUTE, OCH_FABS, OCH_SIGN, OCH_CEIL, OCH_FLOOR, OCH_TRUNC, OCH_ROUND,
   OCH_ISINF, OCH_ISNAN, OCH_ISFINITE, OCH_ISPOSINF, OCH_ISNEGINF,
   OCH_UNARY_COUNT
} och_unary_op;

int och_unary(int op, int dtype, int ndims, const size_t *size,
              const ptrdiff_t *strides1, void *ptr1,
              const ptrdiff_t *strides2, void *ptr2, och_stream stream);
int och_unary_supported(int op, int dtype);   /* LUT entry != 0, ocean_solid.h:131-140 */
int och_unary_result_dtype(int op, int dtype);

/* ======================================================================== */
/* Binary elementwise: z = f(x, y)  (template_binary.cu:35-264)             */
/* Order follows include/ocean/core/generic/generate_tensor_binary.h:19-47. */
/* Operand 2 has type int8 for the bit shifts and int16 for integer/bool    */
/* power (template_binary.cu:201,261); comparisons write bool.              */
/* ptr3/strides3 NULL selects the in-place form z = x.                      */
/* ======================================================================== */
typedef enum {
   OCH_ADD = 0, OCH_SUBTRACT, OCH_MULTIPLY, OCH_DIVIDE, OCH_TRUE_DIVIDE, OCH_FLOOR_DIVIDE,
   OCH_POWER, OCH_MOD, OCH_FMOD,
   OCH_MIN, OCH_MAX, OCH_FMIN, OCH_FMAX,
   OCH_LT, OCH_LE, OCH_EQ, OCH_NE, OCH_GE, OCH_GT,
   OCH_BITWISE_AND, OCH_BITWISE_OR, OCH_BITWISE_XOR,
   OCH_LOGICAL_AND, OCH_LOGICAL_OR, OCH_LOGICAL_XOR,
   OCH_BITSHIFT_LEFT, OCH_BITSHIFT_RIGHT,
   OCH_BINARY_COUNT
} och_binary_op;

int och_binary(int op, int dtype, int ndims, const size_t *size,
               const ptrdiff_t *strides1, void *ptr1,
               const ptrdiff_t *strides2, void *ptr2,
               const ptrdiff_t *strides3, void *ptr3, och_stream stream);
int och_binary_supported(int op, int dtype);
int och_binary_operand2_dtype(int op, int dtype);
int och_binary_result_dtype(int op, int dtype);

/* ======================================================================== */
/* Full reductions (template_reduce_all.cu:54-88; reduce_all.h:365-414)     */
/* One launch; the scalar result is written to host memory at `result` in   */
/* the op's result type and the call returns after the stream has finished  */
/* the reduction (the reference synchronises too, reduce_all.h:404-410).    */
/* Result types (reduce_ops.h): any/all/all_*: bool (uint8); nnz: uint64;   */
/* sum/prod: uint64 | int64 | same float; sum_abs/maximum_abs/minimum_abs/  */
/* norm*: magnitude type (ints: uint64 for sum_abs, unsigned twin for       */
/* max/min abs, double for norms); maximum/minimum: same as input.          */
/* `buffer` may be NULL (the library then uses a per-device scratch block); */
/* otherwise it must hold och_reduce_all_buffer_size() bytes.               */
/* bound/lower/upper are given in the tensor's own dtype.                   */
/* Reductions (full and along axes) read a contiguous row that is not made  */
/* of whole 16-byte groups in ALIGNED 16-byte loads: of the first and last  */
/* 16-byte unit that a row touches, bytes next to the row are loaded too    */
/* (never used, never written). No load leaves a 16-byte unit of which the  */
/* tensor owns at least one byte.                                           */
/* ======================================================================== */
typedef enum {
   OCH_R_ANY = 0, OCH_R_ALL, OCH_R_ALL_FINITE, OCH_R_ANY_INF, OCH_R_ANY_NAN,
   OCH_R_NNZ, OCH_R_NNZ_NAN,
   OCH_R_ALL_LT, OCH_R_ALL_LE, OCH_R_ALL_GT, OCH_R_ALL_GE,
   OCH_R_ALL_GTLT, OCH_R_ALL_GTLE, OCH_R_ALL_GELT, OCH_R_ALL_GELE,
   OCH_R_SUM, OCH_R_SUM_NAN, OCH_R_PROD, OCH_R_PROD_NAN,
   OCH_R_SUM_ABS, OCH_R_SUM_ABS_NAN,
   OCH_R_MAXIMUM, OCH_R_MINIMUM, OCH_R_MAXIMUM_ABS, OCH_R_MINIMUM_ABS,
   OCH_R_NORM, OCH_R_NORM_NAN, OCH_R_NORM2, OCH_R_NORM2_NAN,
   OCH_REDUCE_COUNT
} och_reduce_op;

size_t och_reduce_all_buffer_size(void);     /* solid_gpu_reduce_get_buffer_size, op/reduce_all.c:111-123 */
int och_reduce_supported(int op, int dtype);
int och_reduce_result_dtype(int op, int dtype);
int och_reduce_all(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                   void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                   void *result, void *buffer, och_stream stream);
/* Same reduction, result left in device memory at `dresult`; no host synchronisation. */
int och_reduce_all_device(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                   void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                   void *dresult, void *buffer, och_stream stream);
/* The same reduction for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses */
/* that forbid hipMalloc). No counterpart in the reference. It calls no allocating routine: the partial slots and the */
/* ticket counter live in a fixed array of och_reduce_all_buffer_size() bytes (8448) inside the library's device code, */
/* one copy per device, held until the process ends; its address is looked up by och_device_warmup (or by the first   */
/* call on a device). Tensors of more than och_reduce_all_noalloc_max_elements() (2^40) elements are refused with an  */
/* error. All calls on one device share the array: calls that overlap (different streams, different host threads) on  */
/* one device race and give wrong results; calls on one stream are ordered and safe. */
int och_reduce_all_device_noalloc(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                   void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                   void *dresult, och_stream stream);
size_t och_reduce_all_noalloc_max_elements(void);
/* A full reduction over a layout of several dimensions indexes at most 0xFFFF0000 elements per launch (the reference  */
/* switches to 64-bit indices instead, solid/src/core/gpu/op/apply_elemwise.c:68-99). Larger tensors are cut along     */
/* their outer dimensions into boxes that are launched one after the other; the launches share the partial slots and  */
/* the ticket counter, and the last block of the last launch folds. och_reduce_cut_parts is that cutting, on the host */
/* alone: first index and extent per dimension of every box (ndims values per box, at most max_boxes boxes written),   */
/* returns the number of boxes, or -1 when dimension 0 alone exceeds the limit (it is never cut). Test hook:           */
/* och_reduce_set_part_limit lowers the number of elements per launch (0 restores the default) so that small tensors  */
/* take this path.                                                                                                    */
long long och_reduce_cut_parts(int ndims, const size_t *size, size_t limit, long long max_boxes, size_t *starts, size_t *counts);
void och_reduce_set_part_limit(size_t nelem);

/* ======================================================================== */
/* Axis reductions (template_reduce_axis.cu:54-80; reduce_axis.h:563-597)   */
/* The configuration mirrors solid_gpu_reduce_axis_config: outer dimensions */
/* (size/strides1 for the source, strides2 for the destination) and the     */
/* reduced dimensions (rsize/rstrides into the source), as produced by      */
/* OcSolid_analyzeReduceAxis (ocean_solid.c:382-462).                       */
/* ======================================================================== */
typedef struct {
   int        ndims;                      /* outer (kept) dimensions */
   size_t     size[OCH_MAX_DIMS];
   ptrdiff_t  strides1[OCH_MAX_DIMS];     /* source strides of kept dims */
   ptrdiff_t  strides2[OCH_MAX_DIMS];     /* destination strides */
   int        rdims;                      /* reduced dimensions */
   size_t     rsize[OCH_MAX_DIMS];
   ptrdiff_t  rstrides[OCH_MAX_DIMS];
   void      *ptr1;                       /* source */
   void      *ptr2;                       /* destination, element type = reduce result dtype */
   och_stream stream;
} och_reduce_axis_config;

int och_reduce_axis(int op, int dtype, const och_reduce_axis_config *config, double p);
/* One launch counts its outputs, and the reduced elements of one output, in 32 bits; the reference switches to 64-bit  */
/* indices instead (solid/src/core/gpu/op/apply_elemwise.c:66-99). A reduction with more outputs is cut along its        */
/* outermost kept dimension into pieces that are launched one after the other. A reduced range of more elements is cut  */
/* along its outermost reduced dimension: every piece is a launch that leaves raw accumulators in the stream's workspace */
/* and one finish kernel folds them in the order of the reduced index (a fixed order: results are reproducible). Test   */
/* hooks: the number of outputs and of reduced elements per launch can be lowered (0 restores the default) so that      */
/* small tensors are cut.                                                                                               */
void och_reduce_axis_set_output_limit(size_t outputs);
void och_reduce_axis_set_range_limit(size_t nelem);

/* ======================================================================== */
/* GEMM: C <- alpha * op(A) * op(B) + beta * C, column-major, ld in elements*/
/* Replaces cublas{S,D,C,Z}gemm dispatch (src/core/gpu/op/tensor_blas_gpu.c */
/* :132-231) and solid_gpu_gemm for bool/integers (template_blas.cu:99-237).*/
/* trans in {'N','T','C'}. alpha/beta point to one element of `dtype` in    */
/* host memory (scalar_mode_host != 0) or device memory.                    */
/* bool uses OR/AND arithmetic (template_blas.cu).                          */
/* ======================================================================== */
int och_gemm(int dtype, char transA, char transB, size_t M, size_t N, size_t K,
             const void *alpha, const void *A, ptrdiff_t ldA,
             const void *B, ptrdiff_t ldB,
             const void *beta, void *C, ptrdiff_t ldC,
             int scalar_mode_host, och_stream stream);
int och_gemm_supported(int dtype);
/* The loop over the dimensions beyond the second (tensor_blas_gpu.c:171-252) as one launch: product z of the   */
/* batch is split into indices over batch_size (first dimension fastest) and every operand -- alpha and beta    */
/* included, tensor_blas_gpu.c:236-241 -- moves by its own byte stride per index (0: shared by the products;    */
/* stride_alpha / stride_beta may be NULL for all-zero). nbatch <= 6. The products of a batch must not overlap  */
/* in C. Host scalars that differ between products fall back to one launch per product.                         */
int och_gemm_batched(int dtype, char transA, char transB, size_t M, size_t N, size_t K,
                     const void *alpha, const void *A, ptrdiff_t ldA,
                     const void *B, ptrdiff_t ldB,
                     const void *beta, void *C, ptrdiff_t ldC,
                     int nbatch, const size_t *batch_size,
                     const ptrdiff_t *stride_alpha, const ptrdiff_t *strideA, const ptrdiff_t *strideB,
                     const ptrdiff_t *stride_beta, const ptrdiff_t *strideC,
                     int scalar_mode_host, och_stream stream);

/* Which kernel large aligned float / double / complex-float products take is decided by a cost model (rounds of the   */
/* compute units x tile area / efficiency). For tests and measurements the decision can be fixed: 0 the model decides */
/* (default), 1 the pipelined kernel on its large tile wherever its conditions hold (M, N multiples of 4 or 2, K of   */
/* the slab, 16-byte aligned operands), 2 the pipelined kernel on its small tile (float, double; complex float has    */
/* one tile), 3 never the pipelined kernel, 4 the pipelined kernel on its smallest tile (float: 64 x 64; the other    */
/* types: the tile the model prefers). Process-wide; no counterpart in the reference.                                 */
int och_gemm_set_kernel_choice(int choice);
/* Which kernel the model gives an aligned float product of `batch` entries (0 or 1: a single product) with scalars  */
/* in host memory: 256, 128 or 64 for the pipelined kernel on tiles of that edge, 0 for the tiled kernels. Host      */
/* arithmetic only (no device is touched; without a device the model assumes 256 compute units). No counterpart in   */
/* the reference.                                                                                                     */
int och_gemm_float_plan(size_t M, size_t N, size_t K, unsigned batch);
/* The pipelined kernels' plan for the last round of the compute units, host arithmetic only (no device is touched):   */
/* a product of ceil(M / tile_m) x ceil(N / tile_n) block tiles on `units` compute units, K in slabs of `slab`, every   */
/* element of C elem_size bytes. Returns into how many shares along K each tile of the last round is cut (1: no cut)   */
/* and, in *rounds (may be null), the cost of the product in rounds of whole tiles. No counterpart in the reference.   */
int och_gemm_split_plan(size_t M, size_t N, size_t K, unsigned tile_m, unsigned tile_n, unsigned slab, unsigned elem_size,
                        unsigned units, double *rounds);

/* Fused projection step of a modified Gram-Schmidt sweep. No counterpart in the reference, whose callers issue one    */
/* dot product (gemm with M = N = 1) and one rank-1 update per pair of columns, i.e. 2 k launches for this:             */
/*    for i = 0 .. k-1 (in this order):  r[i] = q_i^H v;   v <- v - r[i] q_i                                            */
/* q_i = Q + i * ldq (ldq in elements) and v are dense vectors of n elements in device memory; r (k elements, device   */
/* memory) receives the coefficients and may be NULL. dtype: OCH_FLOAT, OCH_DOUBLE, OCH_CFLOAT, OCH_CDOUBLE. One launch */
/* for n <= 16384 (the vector stays in the registers of one workgroup); longer vectors run the two gemm launches per    */
/* column and need r. Dot products accumulate in double, as och_gemm's do.                                               */
int och_mgs_project(int dtype, size_t n, size_t k, const void *Q, ptrdiff_t ldq, void *v, void *r, och_stream stream);

/* ======================================================================== */
/* Index operations (template_index.cu:37-57, index1.h:182, index2.h:188)   */
/* ======================================================================== */
int och_add_if_negative(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                        void *ptr, och_scalar value, och_stream stream);
int och_index_to_offset(int dtype, int nstrides, const int64_t *strides, ptrdiff_t stride_reduce,
                        size_t nelem, ptrdiff_t stride1, void *ptr1,
                        ptrdiff_t stride2, void *ptr2, och_stream stream);
int och_get_index(int dtype, int ndims, const size_t *size, int64_t **offsets,
                  const ptrdiff_t *strides1, void *ptr1,
                  const ptrdiff_t *strides2, void *ptr2, och_stream stream);
int och_set_index(int dtype, int ndims, const size_t *size, int64_t **offsets,
                  const ptrdiff_t *strides1, void *ptr1,
                  const ptrdiff_t *strides2, void *ptr2, och_stream stream);
int och_fill_index(int dtype, int ndims, const size_t *size, int64_t **offsets,
                   const ptrdiff_t *strides, void *ptr, och_scalar value, och_stream stream);

/* ======================================================================== */
/* Find / mask-to-offset: positions of the non-zero elements of a bool      */
/* tensor, in the order of its dimensions with dimension 0 running fastest. */
/* The reference has these on the CPU only (solid_cpu_find_prepare, _apply, */
/* _finalize, solid/src/core/cpu/template_index.c:296-500; callers          */
/* src/core/cpu/op/tensor_index_cpu.c:60-155; the GPU table leaves          */
/* Tensor_find and Tensor_maskToOffset empty, docs/future_work.md:33).      */
/*  och_find_count  counts the non-zero elements and fills `workspace`      */
/*                  (device memory, och_find_workspace_size(nelem) bytes)   */
/*                  with per-chunk start positions; returns after the count */
/*                  is known (one stream synchronisation).                  */
/*  och_find_apply  writes, for the k-th non-zero element, either its ndims */
/*                  indices to out[k*ndims .. ] (multiplier == NULL) or the */
/*                  single value sum_d index_d * multiplier[d] to out[k].   */
/* ======================================================================== */
size_t och_find_workspace_size(size_t nelem);
int och_find_count(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                   void *workspace, size_t *nnz, och_stream stream);
int och_find_apply(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                   void *workspace, const int64_t *multiplier, int64_t *out, och_stream stream);

/* ======================================================================== */
/* Launch analysis of an elementwise call, without launching anything.      */
/* Reports what the library derives from the operands before a launch, the  */
/* counterpart of solid_gpu_elemwise{1,2,3}_analyze (src/core/gpu/op/       */
/* apply_elemwise3.c:43-156: drop unit dimensions, sort, merge, pick a      */
/* kernel): the normalised shape (dimensions sorted by the strides of the   */
/* last operand, negative strides of that operand flipped, mergeable        */
/* dimensions merged), the byte offset this adds to each pointer, the       */
/* kernel family, the elements per thread-level access, the number of       */
/* launches, and the multiply-shift constants that replace the division by  */
/* each dimension in the kernels. The last operand is the destination.      */
/* Needs no GPU.                                                            */
/* ======================================================================== */
enum { OCH_KERNEL_WIDE = 0, OCH_KERNEL_MIXED = 1, OCH_KERNEL_SINGLE = 2, OCH_KERNEL_TILED = 3, OCH_KERNEL_ROWS = 4 };
typedef struct {
   int        ndims;
   size_t     size[OCH_MAX_DIMS];
   ptrdiff_t  strides[3][OCH_MAX_DIMS];
   ptrdiff_t  offset[3];
   int        kernel;                     /* OCH_KERNEL_* of the first launch */
   int        vec;                        /* elements per access in that launch */
   int        launches;                   /* kernel launches for the whole call */
   unsigned   div_d[OCH_MAX_DIMS], div_m[OCH_MAX_DIMS], div_s1[OCH_MAX_DIMS], div_s2[OCH_MAX_DIMS];
   unsigned   row_units;                  /* OCH_KERNEL_ROWS: work items per row of dimension 0 */
   size_t     row_elements;               /* OCH_KERNEL_ROWS: elements in such a row */
} och_elemwise_plan;
int och_elemwise_analyze(int noperands, const int *elemsize, int ndims, const size_t *size,
                         const ptrdiff_t *const *strides, void *const *ptrs, och_elemwise_plan *plan);
/* One launch of the elementwise engine (binary, unary, copy / cast / byteswap, fill, steps, the index kernels) counts    */
/* its work items in 32 bits: at most 0xFFFF0000 elements. The reference switches its kernels to 64-bit indices above   */
/* that (solid/src/core/gpu/op/apply_elemwise.c:66-99); here a larger call is cut along its outermost dimension into    */
/* runs that are launched one after the other on the stream (a one-dimensional call into runs of a multiple of 64       */
/* elements), a copy between different shapes along the flat index both sides share, and the gather / scatter kernels   */
/* decompose a 64-bit work-item number. Test hook: the limit can be lowered (64 ... 0xFFFF0000; 0 restores the default) */
/* so that small tensors take these paths; och_elemwise_analyze reports the launches a call would make. Returns -1 for  */
/* a value outside that range.                                                                                          */
int och_elemwise_set_launch_limit(size_t nelem);
/* OCH_KERNEL_ROWS (unit-stride rows that are not whole aligned vectors: an odd width, a start or a pitch that is not  */
/* a multiple of the vector width): a work item is one aligned unit of `vec` elements of a destination row. For unit   */
/* number `unit` of a row of row_elements elements of elemsize bytes that starts `misalignment` bytes into such a unit: */
/* *first = row position of the unit's element 0 (negative in a first unit that begins in front of the row), [lo, hi)  */
/* = its elements inside the row; returns 1 when there are any, else 0. Units with lo = 0 and hi = vec move with one   */
/* access per operand, the others element by element. och_elemwise_row_units: units given to every row.                */
int och_elemwise_row_unit(unsigned unit, int misalignment, int elemsize, int vec, size_t row_elements,
                          long long *first, int *lo, int *hi);
size_t och_elemwise_row_units(size_t row_elements, int elemsize, int vec);

#ifdef __cplusplus
}
#endif
#endif
