/* Object layouts and the core-module function table that Ocean's interface layer and its GPU
 * device module share. These are restatements, field for field, of the reference's public
 * structs, so that code built against this header is layout-compatible with Ocean's libraries:
 *   OcDType                 include/ocean/base/dtype.h:29-36
 *   OcSize/OcIndex, scalars include/ocean/base/types.h:27-46
 *   OcScalar                include/ocean/base/scalar.h:30-63
 *   OcStream/OcEvent/OcDevice include/ocean/base/device.h:81-118
 *   OcStorage               include/ocean/base/storage.h:48-64
 *   OcTensor                include/ocean/base/tensor.h:63-79 (flags :47-51)
 *   OcTensorIndexView       include/ocean/base/index.h:125-130
 *   OcDeviceModule          include/ocean/base/device_module.h:27-38
 *   OcModuleCore            include/ocean/core/interface/module_core.h:43-164
 * (sizes and field offsets are checked against numbers taken from the reference headers:
 * tests/golden/abi_layout.json).
 */
#ifndef OCEAN_ABI_H
#define OCEAN_ABI_H
#include <stddef.h>
#include <stdint.h>

typedef enum
{  OcDTypeBool = 0, OcDTypeUInt8, OcDTypeUInt16, OcDTypeUInt32, OcDTypeUInt64,
   OcDTypeInt8, OcDTypeInt16, OcDTypeInt32, OcDTypeInt64,
   OcDTypeHalf, OcDTypeFloat, OcDTypeDouble, OcDTypeCHalf, OcDTypeCFloat, OcDTypeCDouble,
   OcDTypeNone
} OcDType;
#define OC_DTYPE_COUNT 15
#define OC_TENSOR_MAX_DIMS 8

typedef char OcBool;  typedef int8_t OcInt8;   typedef int16_t OcInt16;   typedef int32_t OcInt32;   typedef int64_t OcInt64;
typedef uint8_t OcUInt8; typedef uint16_t OcUInt16; typedef uint32_t OcUInt32; typedef uint64_t OcUInt64;
typedef uint16_t OcHalf; typedef float OcFloat; typedef double OcDouble;
typedef struct { OcHalf real, imag; } OcCHalf;
typedef struct { OcFloat real, imag; } OcCFloat;
typedef struct { OcDouble real, imag; } OcCDouble;
typedef ptrdiff_t OcIndex;
typedef ptrdiff_t OcSize;

typedef struct
{  OcDType dtype;
   union
   {  OcBool sBool; OcUInt8 sUInt8; OcUInt16 sUInt16; OcUInt32 sUInt32; OcUInt64 sUInt64;
      OcInt8 sInt8; OcInt16 sInt16; OcInt32 sInt32; OcInt64 sInt64;
      OcHalf sHalf; OcFloat sFloat; OcDouble sDouble; OcCHalf sCHalf; OcCFloat sCFloat; OcCDouble sCDouble;
   } value;
} OcScalar;

struct __OcDevice;
typedef struct __OcDeviceType                          /* include/ocean/base/device.h:66-78 */
{  char        *name;
   long int     refcount;
   struct __OcDevice **devices;            /* device instances, not reference counted */
   int          deviceCount;
   char        *lutBuffer;                 /* the registered module tables, one after the other */
   size_t       lutSize;
   size_t       lutCapacity;
} OcDeviceType;
typedef struct __OcModule OcModule;                    /* opaque */

typedef struct __OcStream { struct __OcDevice *device; struct __OcStream *next; long int refcount; } OcStream;
typedef struct __OcEvent  { struct __OcEvent *next; } OcEvent;

typedef struct __OcDevice
{  OcDeviceType *type;
   int           index;
   char         *name;
   int           endianness;               /* 0 little, 1 big */
   int           requiresAlignedData;
   long int      refcount;
   void        **contextBuffer;            /* one context per registered module */
   size_t        contextSize;
   size_t        contextCapacity;
   OcStream     *defaultStream;
   OcStream *(*create_stream)(struct __OcDevice *device);
   int       (*create_event )(struct __OcDevice *device, OcEvent **event);
   void      (*delete_stream)(OcStream *stream);
   void      (*delete_event )(struct __OcDevice *device, OcEvent *event);
   int       (*sync_stream  )(OcStream *stream);
   int       (*sync_event   )(OcEvent *event);
   int       (*record_event )(OcEvent *event, OcStream *stream);
   int       (*wait_event   )(OcStream *stream, OcEvent *event);
   void      (*finalize     )(struct __OcDevice *device);
} OcDevice;

#define OC_STORAGE_OWNER        0x0001
#define OC_STORAGE_RAW          0x0002
#define OC_STORAGE_BYTESWAPPED  0x0004
#define OC_STORAGE_READONLY     0x0008
typedef uint32_t OcStorageFlags;
typedef struct __OcStorage
{  OcStream      *stream;
   OcEvent       *event;
   char          *data;
   OcDType        dtype;
   OcSize         size;                    /* bytes in use */
   OcSize         capacity;                /* bytes allocated */
   OcSize         nelem;
   int            elemsize;
   OcStorageFlags flags;
   long int       refcount;
   void         (*finalize)(struct __OcStorage *storage);
} OcStorage;

#define OC_TENSOR_BYTESWAPPED   0x1000
#define OC_TENSOR_READONLY      0x2000
typedef uint32_t OcTensorFlags;
typedef struct
{  int            ndims;
   int            capacity;
   OcSize        *size;
   OcIndex       *strides;                 /* bytes, signed; 0 = broadcast */
   OcSize         offset;                  /* bytes into the storage */
   OcStorage     *storage;
   OcDevice      *device;
   OcDType        dtype;
   int            elemsize;
   OcSize         nelem;
   OcSize         blockOffset;
   OcSize         blockExtent;
   long int       refcount;
   OcTensorFlags  flags;
} OcTensor;
#define OcTensor_data(t)           ((t)->storage->data + (t)->offset)

typedef struct
{  int        ndims;
   OcTensor  *view;
   OcTensor **offsets;                             /* per dimension: int64 byte offsets, or NULL */
   OcIndex    offsetStrides[OC_TENSOR_MAX_DIMS];
} OcTensorIndexView;

typedef struct __OcDeviceModule
{  OcModule *module;
   void     *data;
   int       available;
   int    (*initializeContext)(OcDevice *device, struct __OcDeviceModule *deviceModule, void **context);
   void   (*finalizeContext  )(OcDevice *device, struct __OcDeviceModule *deviceModule, void *context);
   void   (*finalizeModule   )(struct __OcDeviceModule *deviceModule);
} OcDeviceModule;

#include "oc_op_tables.h"

typedef struct
{  OcDeviceModule HEAD;
   int        (*Device_formatInfo     )(OcDevice *device, char **str, const char *header, const char *footer);
   int        (*Buffer_copy           )(OcStorage *srcStorage, void *srcData, OcStorage *dstStorage, void *dstData, OcDType dtype, OcSize n);
   int        (*Buffer_copyFromCPU    )(OcStorage *srcStorage, void *srcData, OcStorage *dstStorage, void *dstData, OcDType dtype, OcSize n);
   int        (*Buffer_copyToCPU      )(OcStorage *srcStorage, void *srcData, OcStorage *dstStorage, void *dstData, OcDType dtype, OcSize n);
   int        (*Buffer_copyHostStorage)(OcStorage *storage, OcSize offset, OcSize nbytes, void *ptr);
   int        (*Buffer_copyStorageHost)(OcStorage *storage, OcSize offset, OcSize nbytes, void *ptr);
   int        (*Buffer_zero           )(OcStorage *storage, void *data, OcDType dtype, OcSize size);
   OcStorage *(*Storage_create        )(OcSize nelem, OcDType dtype, OcDevice *device, OcStream *stream);
   OcStorage *(*Storage_fromObject    )(OcSize nelem, OcDType dtype, OcDevice *device, void *object, void *data, int byteswapped,
                                        void (*free)(void *object, void *data), OcStream *stream);
   int        (*Tensor_copy           )(OcTensor *src, OcTensor *dst);
   int        (*Tensor_copyFromCPU    )(OcTensor *src, OcTensor *dst);
   int        (*Tensor_copyToCPU      )(OcTensor *src, OcTensor *dst);
   int        (*Tensor_byteswapNoFlag )(OcTensor *tensor);
   int        (*Tensor_fill           )(OcTensor *tensor, OcScalar *scalar);
   int        (*Tensor_fillNaN        )(OcTensor *tensor, OcScalar *scalar);
   int        (*Tensor_maskedFill     )(OcTensor *tensor, OcTensor *mask, OcScalar *scalar);
   int        (*Tensor_stepsInt64     )(OcTensor *tensor, OcInt64 offset, OcInt64 step);
   int        (*Tensor_stepsDouble    )(OcTensor *tensor, OcDouble offset, OcDouble step);
   int        (*Tensor_stepsCDouble   )(OcTensor *tensor, OcCDouble offset, OcCDouble step);
   OcTensor  *(*Tensor_find           )(OcTensor *tensor);
   OcTensor  *(*Tensor_maskToOffset   )(OcTensor *tensor, OcIndex *strides);
   int        (*Tensor_indexToOffset  )(OcTensor *tensor, OcInt64 *strides, OcTensor *offsets);
   int        (*Tensor_addIfNegative  )(OcTensor *tensor, OcScalar *scalar);
   int        (*Tensor_getIndex       )(OcTensorIndexView *view, OcTensor *dst);
   int        (*Tensor_setIndex       )(OcTensorIndexView *view, OcTensor *src);
   int        (*Tensor_fillIndex      )(OcTensorIndexView *view, OcScalar *scalar);
#define OC_X(NAME, OP) int (*Tensor_##NAME)(OcTensor *src, OcTensor *dst);
   OC_UNARY_TABLE(OC_X)
#undef OC_X
#define OC_X(NAME, OP) int (*Tensor_##NAME)(OcTensor *tensor1, OcTensor *tensor2, OcTensor *tensor3);
   OC_BINARY_TABLE(OC_X)
#undef OC_X
   int        (*Tensor_allGELE        )(OcTensor *tensor, OcScalar *lower, OcScalar *upper, int *result);
   int        (*Tensor_allGELT        )(OcTensor *tensor, OcScalar *lower, OcScalar *upper, int *result);
   int        (*Tensor_allGTLE        )(OcTensor *tensor, OcScalar *lower, OcScalar *upper, int *result);
   int        (*Tensor_allGTLT        )(OcTensor *tensor, OcScalar *lower, OcScalar *upper, int *result);
   int        (*Tensor_allLE          )(OcTensor *tensor, OcScalar *bound, int *result);
   int        (*Tensor_allLT          )(OcTensor *tensor, OcScalar *bound, int *result);
   int        (*Tensor_allGE          )(OcTensor *tensor, OcScalar *bound, int *result);
   int        (*Tensor_allGT          )(OcTensor *tensor, OcScalar *bound, int *result);
   int        (*Tensor_any            )(OcTensor *tensor, int *result);
   int        (*Tensor_all            )(OcTensor *tensor, int *result);
   int        (*Tensor_allFinite      )(OcTensor *tensor, int *result);
   int        (*Tensor_anyInf         )(OcTensor *tensor, int *result);
   int        (*Tensor_anyNaN         )(OcTensor *tensor, int *result);
   int        (*Tensor_nnz            )(OcTensor *tensor, OcUInt64 *result);
   int        (*Tensor_nnzNaN         )(OcTensor *tensor, OcUInt64 *result);
   int        (*Tensor_sum            )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_prod           )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_sumNaN         )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_prodNaN        )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_sumAbs         )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_sumAbsNaN      )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_maximum        )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_minimum        )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_maximumAbs     )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_minimumAbs     )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_norm2          )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_norm2NaN       )(OcTensor *tensor, OcScalar *result);
   int        (*Tensor_norm           )(OcTensor *tensor, double p, OcScalar *result);
   int        (*Tensor_normNaN        )(OcTensor *tensor, double p, OcScalar *result);
#define OC_X(NAME, OP) int (*Tensor_##NAME)(OcTensor *src, int n, int *axes, OcTensor *dst);
   OC_AXIS_TABLE(OC_X)
#undef OC_X
   int        (*Tensor_axisNorm       )(OcTensor *src, double p, int n, int *axes, OcTensor *dst);
   int        (*Tensor_axisNormNaN    )(OcTensor *src, double p, int n, int *axes, OcTensor *dst);
   int        (*Tensor_gemm           )(OcSize M, OcSize N, OcSize K, char transA, char transB,
                                        OcTensor *alpha, OcTensor *A, OcIndex ldA, OcTensor *B, OcIndex ldB,
                                        OcTensor *beta, OcTensor *C, OcIndex ldC);
   int        (*Tensor_gemmSupportedOn)(OcDevice *device, OcDType dtype);
} OcModuleCore;

typedef struct
{  OcStorage **bufferList;
   int         bufferCount;
   int         bufferIndex;
   OcSize      bufferMaxSize;
   OcTensor   *scalarList[OC_DTYPE_COUNT][8];
   int         scalarIndex[OC_DTYPE_COUNT];
   int         scalarCount;
} OcModuleCore_Context;

#endif
