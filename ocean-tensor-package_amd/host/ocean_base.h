/* Declarations of the functions of Ocean's base library (libocean_base), of its interface layer (libocean_core) and of
 * the ocean-solid glue that the GPU device module calls, with the reference's names, argument lists and meaning. The
 * stand-in implementations are in host_base.c. Where each comes from in the reference:
 *   errors    include/ocean/base/error.h:30-68, src/base/error.c
 *   memory    include/ocean/base/malloc.h:42-43
 *   dtype     include/ocean/base/dtype.h, src/base/dtype.c:88-178
 *   devices   include/ocean/base/device.h:127-181, src/base/device.c
 *   modules   include/ocean/base/device_module.h:47, src/base/device_module.c:313-422; include/ocean/core/interface/module_core.h:177-186
 *   storage   include/ocean/base/storage.h:72-101, src/base/storage.c:36-222; include/ocean/core/interface/storage_itf.h:31-33
 *   tensors   include/ocean/base/tensor.h:92-169, include/ocean/core/interface/tensor_itf.h:49-53
 *   shapes    include/ocean/base/shape.h:27-45
 *   solid     include/ocean/external/ocean-solid/ocean_solid.h:73-83,120
 */
#ifndef OCEAN_BASE_H
#define OCEAN_BASE_H
#include "ocean_abi.h"
#include <stdio.h>
#include <stdlib.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- errors ---- */
char       *OcError_getBuffer(void);
size_t      OcError_getBufferSize(void);
void        OcError_setSource(const char *file, size_t line);
const char *OcError_lastError(void);
#define OcErrorMessage(...) do { OcError_setSource(__FILE__, __LINE__); snprintf(OcError_getBuffer(), OcError_getBufferSize(), __VA_ARGS__); } while (0)
#define OcError(CODE, ...)  do { OcErrorMessage(__VA_ARGS__); return (CODE); } while (0)

/* ---- memory ---- */
#define OcMalloc malloc
#define OcFree   free

/* ---- finalisation (include/ocean/base/ocean.h:27) ---- */
int  OcFinalizeAddHandler(void (*funptr)(void), const char *desc);
void OcFinalize(void);                                  /* runs the handlers, last added first */

/* ---- dtype ---- */
int     OcDType_size(OcDType dtype);
int     OcDType_isFloat(OcDType dtype);     /* half, float, double and the complex types */
int     OcDType_isComplex(OcDType dtype);
int     OcDType_isSigned(OcDType dtype);
OcDType OcDType_getBaseType(OcDType dtype);
OcDType OcDType_getCommonType(OcDType dtype1, OcDType dtype2);
const char *OcDType_name(OcDType dtype);

/* ---- devices, streams, events ---- */
extern OcDevice *OcCPU;
OcDeviceType *OcCreateDeviceType(const char *name);
OcDeviceType *OcIncrefDeviceType(OcDeviceType *deviceType);
void          OcDecrefDeviceType(OcDeviceType *deviceType);
OcDeviceType *OcDeviceTypeByName(const char *name);
OcDevice     *OcCreateDevice(OcDeviceType *type, int index, const char *name, size_t size);
int           OcRegisterDevice(OcDevice *device);
OcDevice     *OcIncrefDevice(OcDevice *device);
void          OcDecrefDevice(OcDevice *device);
OcStream     *OcIncrefStream(OcStream *stream);
void          OcDecrefStream(OcStream *stream);
OcStream     *OcDevice_createStream(OcDevice *device);
int           OcStream_synchronize(OcStream *stream);
int           OcStream_waitFor(OcStream *stream, OcEvent *event);
int           OcDevice_createEvent(OcDevice *device, OcEvent **event);
void          OcDevice_freeEvent(OcDevice *device, OcEvent *event);
int           OcEvent_synchronize(OcDevice *device, OcEvent *event);
int           OcEvent_record(OcEvent *event, OcStream *stream);

/* ---- device modules ---- */
extern OcModule oc_module_core;                                             /* include/ocean/core/interface/module_core.h:173 */
int  OcRegisterModule(const char *deviceType, OcDeviceModule *info, size_t size);
int  OcModuleCore_initialize(void);
OcModuleCore_Context *OcModuleCore_createContext(OcDevice *device, size_t size);
void                  OcModuleCore_freeContext(OcModuleCore_Context *context);
OcModuleCore_Context *OcModuleCore_getContext(OcDevice *device);

/* ---- storage ---- */
OcStorage *OcAllocateStorage(OcDevice *device, OcDType dtype, OcStream *stream, OcSize size);
OcStorage *OcIncrefStorage(OcStorage *storage);
void       OcDecrefStorage(OcStorage *storage);
int        OcStorage_isOwner(OcStorage *storage);
int        OcStorage_synchronize(OcStorage *storage);
int        OcStorage_update(OcStorage *storage);
int        OcStorage_startRead(OcStorage *storage, OcStorage *readStorage);
int        OcStorage_finishRead(OcStorage *storage, OcStorage *readStorage);
int        OcStorage_startWrite(OcStorage *storage, OcStorage *writeStorage);
int        OcStorage_finishWrite(OcStorage *storage, OcStorage *writeStorage);
OcStorage *OcStorage_create(OcSize nElements, OcDType dtype, OcDevice *device);
OcStorage *OcStorage_createTemporary(OcSize nElements, OcDType dtype, OcDevice *device);
OcStorage *OcStorage_createWithStream(OcSize nElements, OcDType dtype, OcStream *stream);

/* ---- tensors ---- */
#define OcTensor_startRead(T, R)   OcStorage_startRead((T)->storage, (R)->storage)
#define OcTensor_finishRead(T, R)  OcStorage_finishRead((T)->storage, (R)->storage)
#define OcTensor_startWrite(T, W)  OcStorage_startWrite((T)->storage, (W)->storage)
#define OcTensor_finishWrite(T, W) OcStorage_finishWrite((T)->storage, (W)->storage)
#define OcTensor_update(T)         OcStorage_update((T)->storage)
#define OcTensor_synchronize(T)    OcStorage_synchronize((T)->storage)
OcTensor *OcTensor_create(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcDevice *device);  /* strides NULL: column-major */
OcTensor *OcTensor_createTemporary(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcDevice *device);
OcTensor *OcTensor_createWithStream(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcStream *stream);
OcTensor *OcTensor_createFromStorage(OcStorage *storage, int ndims, OcSize *size, OcIndex *strides, OcIndex offset, OcDType dtype);
OcTensor *OcTensor_shallowCopy(OcTensor *tensor);
OcTensor *OcIncrefTensor(OcTensor *tensor);
void      OcDecrefTensor(OcTensor *tensor);
int       OcTensor_extent(OcTensor *tensor, OcSize *offset, OcSize *extent);
int       OcTensor_isByteswapped(OcTensor *tensor);
int       OcTensor_isContiguous(OcTensor *tensor);
void      OcTensor_setByteswapped(OcTensor *tensor, int flag);

/* ---- shapes ---- */
int  OcShape_extent(int ndims, OcSize *size, OcIndex *strides, OcSize elemsize, OcSize *dataOffset, OcSize *dataExtent);
void OcShape_sortStrides2(int ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2);
void OcShape_mergeBlocks2(int *ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2);

/* ---- ocean-solid glue ---- */
typedef struct
{  int      ndims;
   int      rdims;
   size_t   size[OC_TENSOR_MAX_DIMS];
   size_t   rsize[OC_TENSOR_MAX_DIMS];
   ptrdiff_t strides1[OC_TENSOR_MAX_DIMS];
   ptrdiff_t strides2[OC_TENSOR_MAX_DIMS];
   ptrdiff_t rstrides[OC_TENSOR_MAX_DIMS];
   void    *ptr1;
   void    *ptr2;
} OcSolidReduceAxis;
void OcSolid_analyzeReduceAxis(OcSolidReduceAxis *config, OcTensor *src, OcTensor *dst, int n, int *axes, int flagRemoveRepeats);

/* ---- only in the stand-in: the registered core-module table of a device (what OC_GET_CORE_FUNCTION resolves against),
        sizes and field offsets of the shared structs as a JSON object (layout self-check) ---- */
OcModuleCore *OcModuleCore_forDevice(OcDevice *device);
const char   *OcHost_abiLayout(void);

#ifdef __cplusplus
}
#endif
#endif
