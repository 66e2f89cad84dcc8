/* A small device-independent front end over the module table, for tests, the smoke check and the Python surface:
 * what Ocean's interface layer does before it reaches a device function (common type, automatic casts, broadcasting,
 * byte-order normalisation, GEMM operand preparation), restricted to what those exercise. Implemented in
 * core_interface.c (and the views in host_base.c) after src/core/interface/tensor_itf.c (copy :777-1041,
 * ensure :1226-1304, binary :3983-4133, reductions :5299-5514, axis :5522-5766, gemm :5951-6778) and
 * src/core/generic/tensor_op.c:141-423. Operations are selected by their index in the table's unary / binary block,
 * where the reference has one function per name; the names below are therefore NOT the reference's signatures and
 * this header is never seen by the device module (host/gpu_module.c).
 */
#ifndef CORE_INTERFACE_H
#define CORE_INTERFACE_H
#include "ocean_base.h"

#ifdef __cplusplus
extern "C" {
#endif

const char *OcError_lastMessage(void);                                                  /* = OcError_lastError */

OcTensor *OcTensor_transpose(OcTensor *tensor);                                   /* view: dimensions 0 and 1 exchanged */
OcTensor *OcTensor_slice(OcTensor *tensor, int axis, OcSize start, OcSize count, OcIndex step);   /* view */
OcTensor *OcTensor_broadcastTo(OcTensor *tensor, int ndims, const OcSize *size);  /* view with zero strides */

int OcTensor_copy(OcTensor *src, OcTensor *dst);                                   /* any device, dtype, byte order */
int OcTensor_ensure(OcTensor **tensor, OcDType dtype, OcDevice *device);           /* replaces *tensor by a converted native-order copy when needed */
int OcTensor_fill(OcTensor *tensor, OcScalar *value);
int OcTensor_fillNaN(OcTensor *tensor, OcScalar *value);                           /* value converted to the tensor's type */
int OcTensor_maskedFill(OcTensor *tensor, OcTensor *mask, OcScalar *value);        /* mask: any type / device, broadcast to the tensor */
int OcTensor_stepsInt64(OcTensor *tensor, OcInt64 offset, OcInt64 step);           /* value(i) = offset + i * step, flat index */
int OcTensor_stepsDouble(OcTensor *tensor, OcDouble offset, OcDouble step);
OcTensor *OcTensor_find(OcTensor *mask);                                         /* ndims x nnz indices of the non-zero elements */
OcTensor *OcTensor_maskToOffset(OcTensor *mask, OcIndex *strides);               /* nnz offsets sum(index * strides) */
int OcTensor_binary(int op, OcTensor *src1, OcTensor *src2, OcTensor **dst);       /* op: index into the table's binary block */
int OcTensor_unary(int op, OcTensor *src, OcTensor **dst);
int OcTensor_reduceAll(int which, OcTensor *tensor, double p, OcScalar *result);    /* which: och reduction index of an OcScalar-valued reduction */
int OcTensor_reduceLogical(int which, OcTensor *tensor, int *result);            /* which: 0 any, 1 all, 2 allFinite, 3 anyInf, 4 anyNaN */
int OcTensor_reduceCount(int which, OcTensor *tensor, OcUInt64 *result);         /* which: 5 nnz, 6 nnzNaN */
int OcTensor_axisReduce(int which, OcTensor *src, int n, int *axes, int keepdims, double p, OcTensor **dst);
int OcTensor_gemm(OcScalar *alpha, OcTensor *A, char modeA, OcTensor *B, char modeB, OcScalar *beta, OcTensor **C);
int OcTensor_gemmTensors(OcTensor *alpha, OcTensor *A, char modeA, OcTensor *B, char modeB, OcTensor *beta, OcTensor **C);   /* scalars as tensors (one per product), NULL: 1 and 0 */
int OcTensor_mtimes(OcTensor *A, OcTensor *B, OcTensor **C);
/* index operations through the table: indices is an int64 tensor of shape [nindexed dims, n]; view dimensions beyond it stay whole */
int OcTensor_getIndexed(OcTensor *tensor, OcTensor *indices, OcTensor **dst);
int OcTensor_setIndexed(OcTensor *tensor, OcTensor *indices, OcTensor *src);

#ifdef __cplusplus
}
#endif
#endif
