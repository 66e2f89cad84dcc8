/* ------------------------------------------------------------------------ */
/* ocean_gpu_module.h -- what the GPU device module built on ocean_hip.h     */
/* exports under the reference's own names: the entry points that Ocean's    */
/* package initialisation and its Python layer bind (include/ocean_gpu.h,    */
/* include/ocean/core/gpu/device_gpu.h). The module itself is                 */
/* ocean-tensor-package_amd/host/gpu_module.c; it is written against Ocean's  */
/* base API only, so it builds against the reference's headers and links      */
/* against libocean_base / libocean_core as src/core/gpu does.                */
/*                                                                          */
/* Include after Ocean's headers ("ocean.h") -- or after host/ocean_abi.h    */
/* where Ocean's headers are not present: OcDevice and OcTensor must be       */
/* declared.                                                                 */
/* ------------------------------------------------------------------------ */
#ifndef OCEAN_GPU_MODULE_H
#define OCEAN_GPU_MODULE_H

#ifdef __cplusplus
extern "C" {
#endif

/* include/ocean/core/gpu/device_gpu.h:31-106. The properties of a GPU device under the reference's field names, so that
   code that reads them (interfaces/python/pyOcean/gpu/pyOcean_device_gpu.c:181-420) compiles unchanged. Filled from the
   HIP device properties: warpSize is the wavefront size (64), major.minor the gfx number (9.5), multiProcessorCount
   the number of compute units, sharedMemPerBlock the LDS a workgroup may use. Fields CUDA-only parts report (tccDriver,
   the unified / managed memory flags, the single-to-double ratio) are zero. */
typedef struct
{  char   name[256];
   size_t totalGlobalMem;
   size_t freeGlobalMem;                 /* refreshed by OcDeviceGPU_updateProperties */
   size_t sharedMemPerBlock;
   int    regsPerBlock, warpSize;
   size_t memPitch;
   int    maxThreadsPerBlock, maxThreadsDim[3], maxGridSize[3], clockRate;
   size_t totalConstMem;
   int    major, minor, deviceOverlap, multiProcessorCount, kernelExecTimeoutEnabled, integrated, canMapHostMemory, computeMode;
   int    concurrentKernels, ECCEnabled, pciBusID, pciDeviceID, pciDomainID, tccDriver, asyncEngineCount, unifiedAddressing;
   int    memoryClockRate, memoryBusWidth, l2CacheSize, maxThreadsPerMultiProcessor, streamPrioritiesSupported;
   int    globalL1CacheSupported, localL1CacheSupported;
   size_t sharedMemPerMultiprocessor;
   int    regsPerMultiprocessor, managedMemSupported, isMultiGpuBoard, multiGpuBoardGroupID;
   int    singleToDoublePrecisionPerfRatio, pageableMemoryAccess, concurrentManagedAccess, hostNativeAtomicSupported;
   int    maxBlocksPerMultiProcessor, maxWarpsPerMultiProcessor, maxSharedMemPerSM;
} OcDevicePropGPU;

/* device_gpu.h:109-120: a GPU device is an OcDevice followed by its properties and the free lists of recycled streams
   and events (at most 64 each, device_gpu.c:251-370); what lies behind them belongs to the module */
typedef struct
{  OcDevice        HEAD;
   OcDevicePropGPU properties;
   OcStream       *streamBuffer;
   OcEvent        *eventBuffer;
   int             streamCount;
   int             eventCount;
} OcDeviceGPU;

/* src/core/gpu/ocean_gpu.c:38-58: idempotent; creates the "GPU" device type and one device per HIP device (device_gpu.c:196-250),
   fills the core-module table and registers it (module_core_gpu.c:127-145), registers OcFinalizeGPU with Ocean's finalisation */
int  OcInitGPU(void);
void OcFinalizeGPU(void);                                          /* ocean_gpu.c:62-72 */

extern OcDevice **OcGPU;                                           /* device_gpu.c:44: OcGPU[i], i < OcDeviceGPUCount() */
int       OcDeviceGPUCount(void);                                  /* device_gpu.h:151, device_gpu.c:429-433 */
OcDevice *OcDeviceGPUByIndex(int index);                           /* device_gpu.h:152, device_gpu.c:437-443: NULL when out of range */
int       OcDeviceGPU_peerAccess(int device1, int device2);        /* device_gpu.h:153, device_gpu.c:447-454 */
int       OcDeviceGPU_isInstance(OcDevice *device);                /* device_gpu.h:154, device_gpu.c:458-462 */
int       OcDeviceGPU_updateProperties(OcDeviceGPU *device);       /* device_gpu.h:157, device_gpu.c:620-637: refreshes freeGlobalMem; 0 or -1 */
int       OcInitDevicesGPU(void);                                  /* device_gpu.h:160, device_gpu.c:196-250: device type + devices */
int       OcInitModuleCore_GPU(void);                              /* module_core_gpu.h:39, module_core_gpu.c:127-145: fills and registers the table */

/* The pieces OcInitModuleCore_GPU assembles the table from (module_core_gpu.c:40-63); each sets its entries of `module` */
int  OcRegisterDevicesGPU(OcModuleCore *module);                   /* device_info.h:29: Device_formatInfo */
int  OcRegisterStorageGPU(OcModuleCore *module);                   /* storage_gpu.h:43: Storage_create and the Buffer_* entries */
int  OcRegisterTensorGPU(OcModuleCore *module);                    /* tensor_gpu.h:30: the nine groups below */
void OcTensorGPU_initializeCopyOps(OcModuleCore *module);          /* op/tensor_copy_gpu.h:27 */
void OcTensorGPU_initializeFillOps(OcModuleCore *module);          /* op/tensor_fill_gpu.h:27 */
void OcTensorGPU_initializeStepOps(OcModuleCore *module);          /* op/tensor_steps_gpu.h:27 */
void OcTensorGPU_initializeIndexOps(OcModuleCore *module);         /* op/tensor_index_gpu.h:27 (also find / maskToOffset, empty in the reference) */
void OcTensorGPU_initializeUnaryOps(OcModuleCore *module);         /* op/tensor_unary_gpu.h:26 */
void OcTensorGPU_initializeBinaryOps(OcModuleCore *module);        /* op/tensor_binary_gpu.h:27 */
void OcTensorGPU_initializeBlasOps(OcModuleCore *module);          /* op/tensor_blas_gpu.h:27 */
void OcTensorGPU_initializeReduceAllOps(OcModuleCore *module);     /* op/tensor_reduce_all_gpu.h:27 */
void OcTensorGPU_initializeReduceAxisOps(OcModuleCore *module);    /* op/tensor_reduce_axis_gpu.h:27 */

/* storage_gpu.h:47-55, storage_gpu.c:104-302: the table's Buffer_* entries. Copies between a GPU storage and the host
   block (they wait for the storage's outstanding work first); copies on the device and zero are asynchronous on the
   destination storage's stream and follow the read / write protocol of storage.c:141-222 */
int OcBufferGPU_copy             (OcStorage *srcStorage, void *srcData, OcStorage *dstStorage, void *dstData, OcDType dtype, OcSize n);
int OcBufferGPU_copyFromCPU      (OcStorage *srcStorage, void *srcData, OcStorage *dstStorage, void *dstData, OcDType dtype, OcSize n);
int OcBufferGPU_copyToCPU        (OcStorage *srcStorage, void *srcData, OcStorage *dstStorage, void *dstData, OcDType dtype, OcSize n);
int OcBufferGPU_copyHostToStorage(OcStorage *storage, OcIndex offset, OcSize nbytes, void *ptr);
int OcBufferGPU_copyStorageToHost(OcStorage *storage, OcIndex offset, OcSize nbytes, void *ptr);
int OcBufferGPU_zero             (OcStorage *storage, void *data, OcDType dtype, OcSize n);

/* No counterpart in the reference (its Python layer reads OcDeviceGPU.properties directly): the properties as the device
   library reports them, an och_device_prop of include/ocean_hip.h (architecture name, LDS and cache sizes, clock rates),
   with the amount of free memory refreshed at every call */
int       OcDeviceGPU_properties(OcDevice *device, void *och_device_prop_out);

/* Beside the module table, no counterpart in the reference: v <- v - sum_i q_i (q_i^H v), the columns of Q in order, in one
   launch (och_mgs_project). Q: n x k with dense columns, v: n, r: k or NULL (receives the coefficients); same GPU, same type. */
int       OcTensorGPU_projectColumns(OcTensor *Q, OcTensor *v, OcTensor *r);

#ifdef __cplusplus
}
#endif
#endif
