/* A minimal stand-in for the parts of Ocean's base library and interface layer that surround the
 * GPU device module, so that the module's function table can be driven exactly as Ocean drives
 * it when Ocean's own libraries are not present: error messages, devices, streams, events,
 * storages, tensors (views over storages), the stream synchronisation protocol, and a small
 * interface layer (common type, automatic casts, broadcasting, byte-order normalisation,
 * GEMM operand preparation). Names and argument meanings follow the reference:
 *   errors    include/ocean/base/error.h:57-68
 *   tensors   src/base/tensor.c, src/core/interface/tensor_itf.c (copy :777-1041, ensure :1226-1304,
 *             binary :3983-4133, reductions :5299-5514, axis :5522-5766, gemm :5951-6778)
 *   operator  src/core/generic/tensor_op.c:141-423
 */
#ifndef OCEAN_HOST_H
#define OCEAN_HOST_H
#include "ocean_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- errors ---- */
int         OcErrorMessage(const char *fmt, ...);        /* stores the message, returns -1 */
const char *OcError_lastMessage(void);
#define OcError(code, ...) do { OcErrorMessage(__VA_ARGS__); return (code); } while (0)

/* ---- dtype ---- */
int     OcDType_size(OcDType dtype);
int     OcDType_isFloat(OcDType dtype);     /* half, float, double and the complex types */
int     OcDType_isComplex(OcDType dtype);
int     OcDType_isSigned(OcDType dtype);
OcDType OcDType_getBaseType(OcDType dtype);
OcDType OcDType_getCommonType(OcDType dtype1, OcDType dtype2);
const char *OcDType_name(OcDType dtype);

/* ---- devices ---- */
extern OcDevice  *OcCPU;
extern OcDevice **OcGPU;                    /* OcGPU[i], i < OcDeviceGPUCount() */
int  OcInitGPU(void);                       /* ocean_gpu.c:38-58: idempotent; creates devices, fills and registers the table */
void OcFinalizeGPU(void);
int  OcDeviceGPUCount(void);
OcDevice *OcDeviceGPUByIndex(int index);   /* device_gpu.c:437-443: NULL when out of range */
int  OcDeviceGPU_isInstance(OcDevice *device);                       /* device_gpu.c:458-462 */
int  OcDeviceGPU_peerAccess(int device1, int device2);               /* device_gpu.c:447-454 */
/* device_gpu.c:471-637: the cached properties of a GPU device, with the amount of free memory refreshed (updateProperties) */
int  OcDeviceGPU_properties(OcDevice *device, void *och_device_prop_out);
/* beside the module table (no counterpart in the reference): v <- v - sum_i q_i (q_i^H v), columns in order; r may be NULL */
int  OcTensorGPU_projectColumns(OcTensor *Q, OcTensor *v, OcTensor *r);
OcModuleCore *OcModuleCore_forDevice(OcDevice *device);   /* what OC_GET_CORE_FUNCTION resolves against */
int  OcRegisterModule(const char *deviceType, OcDeviceModule *info, size_t size);

/* ---- storage and tensors ---- */
OcStorage *OcStorage_create(OcSize nelem, OcDType dtype, OcDevice *device);
OcStorage *OcIncrefStorage(OcStorage *storage);
void       OcDecrefStorage(OcStorage *storage);
int        OcStorage_startRead(OcStorage *target, OcStorage *read);
int        OcStorage_finishRead(OcStorage *target, OcStorage *read);
int        OcStorage_update(OcStorage *storage);
int        OcStorage_synchronize(OcStorage *storage);
#define OcTensor_startRead(T, R)   OcStorage_startRead((T)->storage, (R)->storage)
#define OcTensor_finishRead(T, R)  OcStorage_finishRead((T)->storage, (R)->storage)
#define OcTensor_update(T)         OcStorage_update((T)->storage)
#define OcTensor_synchronize(T)    OcStorage_synchronize((T)->storage)

OcTensor *OcTensor_create(int ndims, const OcSize *size, const OcIndex *strides, OcDType dtype, OcDevice *device);  /* strides NULL: Fortran order */
OcTensor *OcTensor_createFromStorage(OcStorage *storage, int ndims, const OcSize *size, const OcIndex *strides, OcSize offset, OcDType dtype);
OcTensor *OcTensor_shallowCopy(OcTensor *tensor);
OcTensor *OcIncrefTensor(OcTensor *tensor);
void      OcDecrefTensor(OcTensor *tensor);
OcTensor *OcTensor_transpose(OcTensor *tensor);                                   /* view: dimensions 0 and 1 exchanged */
OcTensor *OcTensor_slice(OcTensor *tensor, int axis, OcSize start, OcSize count, OcIndex step);   /* view */
OcTensor *OcTensor_broadcastTo(OcTensor *tensor, int ndims, const OcSize *size);  /* view with zero strides */
void      OcTensor_setByteswapped(OcTensor *tensor, int flag);                     /* marks the data as stored in the other byte order */
int       OcTensor_isContiguous(OcTensor *tensor);

/* ---- interface layer (device independent front end) ---- */
int OcTensor_copy(OcTensor *src, OcTensor *dst);                                   /* any device, dtype, byte order */
int OcTensor_ensure(OcTensor **tensor, OcDType dtype, OcDevice *device);           /* replaces *tensor by a converted native-order copy when needed */
int OcTensor_fill(OcTensor *tensor, OcScalar *value);
OcTensor *OcTensor_find(OcTensor *mask);                                         /* ndims x nnz indices of the non-zero elements */
OcTensor *OcTensor_maskToOffset(OcTensor *mask, OcIndex *strides);               /* nnz offsets sum(index * strides) */
int OcTensor_binary(int op, OcTensor *src1, OcTensor *src2, OcTensor **dst);       /* op: index into the table's binary block */
int OcTensor_unary(int op, OcTensor *src, OcTensor **dst);
#define OcTensor_add(a, b, dst)       OcTensor_binary(0, a, b, dst)
#define OcTensor_subtract(a, b, dst)  OcTensor_binary(1, a, b, dst)
#define OcTensor_scale(a, b, dst)     OcTensor_binary(2, a, b, dst)
int OcTensor_sum(OcTensor *tensor, OcScalar *result);
int OcTensor_maximum(OcTensor *tensor, OcScalar *result);
int OcTensor_norm2(OcTensor *tensor, OcScalar *result);
int OcTensor_reduceAll(int which, OcTensor *tensor, double p, OcScalar *result);    /* which: och reduction index of an OcScalar-valued reduction */
int OcTensor_axisReduce(int which, OcTensor *src, int n, int *axes, int keepdims, double p, OcTensor **dst);
int OcTensor_gemm(OcScalar *alpha, OcTensor *A, char modeA, OcTensor *B, char modeB, OcScalar *beta, OcTensor **C);
int OcTensor_mtimes(OcTensor *A, OcTensor *B, OcTensor **C);

/* ---- caller-side analysis (src/external/ocean-solid/ocean_solid.c:382-462, src/base/shape.c:199-411) ---- */
typedef struct
{  int     ndims;  OcSize size[OC_TENSOR_MAX_DIMS];  OcIndex strides1[OC_TENSOR_MAX_DIMS], strides2[OC_TENSOR_MAX_DIMS];
   int     rdims;  OcSize rsize[OC_TENSOR_MAX_DIMS]; OcIndex rstrides[OC_TENSOR_MAX_DIMS];
   OcIndex offset1, offset2;          /* to add to the source / destination data pointers (flipped negative strides) */
} OcSolidReduceAxis;
int OcSolid_analyzeReduceAxis(OcTensor *src, int n, const int *axes, OcTensor *dst, OcSolidReduceAxis *config);
int OcShape_sortStrides2(int ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2);   /* ascending |strides1| */
int OcShape_mergeBlocks2(int *ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2);

/* sizes and field offsets of the shared structs as a JSON object (layout self-check) */
const char *OcHost_abiLayout(void);

#ifdef __cplusplus
}
#endif
#endif
