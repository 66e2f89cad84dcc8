/* The "GPU" device module of Ocean's core module on top of libocean_hip.so.
 *
 * Mirrors src/core/gpu: OcInitGPU (ocean_gpu.c:38-58), device / stream / event objects with
 * free lists (device_gpu.c:81-420), storage (storage_gpu.c:61-302), module registration
 * (module_core_gpu.c:40-145) and one glue function per table entry (the files under src/core/gpu/op).
 * Every glue function activates the device, runs the stream protocol the reference runs and makes
 * ONE call into the device library; function-table lookups by data type become the
 * (operation, dtype) arguments of that call, and a missing table entry becomes an error from
 * och_*_supported.
 */
#include "ocean_host.h"
#include "../../include/ocean_hip.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ---- device objects (device_gpu.c:81-122, 251-420) ------------------------------------ */
#define OC_GPU_MAX_FREE 64                       /* free-list bound, device_gpu.c:251-370 */
typedef struct { OcStream HEAD; och_stream handle; } OcStreamGPU;
typedef struct { OcEvent HEAD; och_event handle; } OcEventGPU;
typedef struct { OcStorage HEAD; } OcStorageGPU;
/* the module's device object: the public part (OcDeviceGPU of include/ocean_gpu_module.h: properties under the
   reference's names, free lists) followed by what only this file uses */
typedef struct
{  OcDeviceGPU     pub;
   och_device_prop hip;                                                /* as the device library reports them */
   long            eventsRecorded, eventsWaited, streamsCreated;      /* activity counters (OcDeviceGPU_activity) */
} OcDeviceGPUFull;
#define freeStreams  pub.streamBuffer
#define nFreeStreams pub.streamCount
#define freeEvents   pub.eventBuffer
#define nFreeEvents  pub.eventCount
/* the context of the core module on a GPU device: the interface's part first (module_core_gpu.h:28-32 has the BLAS
   handle behind it; the MFMA GEMM kernels need none) */
typedef struct { OcModuleCore_Context HEAD; int deviceIndex; } OcModuleCoreGPU_Context;

OcDevice **OcGPU = NULL;
static int oc_gpu_count = 0;
static int oc_gpu_initialized = 0;
static OcDeviceType *oc_device_type_gpu = NULL;
static OcModuleCore oc_module_core_gpu;          /* the table that registration copies (device_module.c:415) */

#define OCH_CALL(x) do { if ((x) != 0) OcError(-1, "%s", och_last_error()); } while (0)
#define GPU_STREAM(t) (((OcStreamGPU *)((t)->storage->stream))->handle)
static int activate(OcDevice *device) { if (och_device_set(device->index) != 0) OcError(-1, "%s", och_last_error()); return 0; }

static OcStream *OcDeviceGPU_createStream(OcDevice *device)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device; OcStreamGPU *s;
   if (g->freeStreams)
   {  s = (OcStreamGPU *)g->freeStreams; g->freeStreams = s->HEAD.next; g->nFreeStreams--; }
   else
   {  if (activate(device) != 0) return NULL;
      s = (OcStreamGPU *)OcMalloc(sizeof(OcStreamGPU));
      if (s == NULL) OcError(NULL, "Insufficient memory to allocate a stream object");
      if (och_stream_create(&s->handle) != 0) { OcErrorMessage("%s", och_last_error()); OcFree(s); return NULL; }
      g->streamsCreated++;
   }
   s->HEAD.device = device; s->HEAD.next = NULL; s->HEAD.refcount = 1;
   return &s->HEAD;
}
/* called by OcDecrefStream when the last reference goes (device.c:225-236, after synchronising the stream) */
static void OcDeviceGPU_deleteStream(OcStream *stream)
{  OcDeviceGPUFull *g;
   if (stream == NULL) return;
   g = (OcDeviceGPUFull *)stream->device;
   if (g->nFreeStreams < OC_GPU_MAX_FREE)
   {  /* a retired stream keeps its small reduction scratch but gives its 64 MB workspace back to the pool */
      och_device_set(stream->device->index);
      och_stream_release_workspace(((OcStreamGPU *)stream)->handle);
      stream->next = g->freeStreams; g->freeStreams = stream; g->nFreeStreams++;
   }
   else { och_stream_destroy(((OcStreamGPU *)stream)->handle); OcFree(stream); }
}
static int OcDeviceGPU_createEvent(OcDevice *device, OcEvent **event)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device; OcEventGPU *e;
   if (g->freeEvents) { e = (OcEventGPU *)g->freeEvents; g->freeEvents = e->HEAD.next; g->nFreeEvents--; }
   else
   {  if (activate(device) != 0) return -1;
      e = (OcEventGPU *)OcMalloc(sizeof(OcEventGPU));
      if (e == NULL) OcError(-1, "Insufficient memory to allocate an event object");
      if (och_event_create(&e->handle, 0) != 0) { OcFree(e); OcError(-1, "%s", och_last_error()); }
   }
   e->HEAD.next = NULL; *event = &e->HEAD;
   return 0;
}
static void OcDeviceGPU_deleteEvent(OcDevice *device, OcEvent *event)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device;
   if (event == NULL) return;
   if (g->nFreeEvents < OC_GPU_MAX_FREE) { event->next = g->freeEvents; g->freeEvents = event; g->nFreeEvents++; }
   else { och_event_destroy(((OcEventGPU *)event)->handle); OcFree(event); }
}
static int OcStreamGPU_synchronize(OcStream *s)  { OCH_CALL(och_stream_synchronize(((OcStreamGPU *)s)->handle)); return 0; }
static int OcEventGPU_synchronize(OcEvent *e)    { OCH_CALL(och_event_synchronize(((OcEventGPU *)e)->handle)); return 0; }
static int OcEventGPU_record(OcEvent *e, OcStream *s)
{  ((OcDeviceGPUFull *)s->device)->eventsRecorded++;
   OCH_CALL(och_event_record(((OcEventGPU *)e)->handle, ((OcStreamGPU *)s)->handle)); return 0;
}
static int OcStreamGPU_waitEvent(OcStream *s, OcEvent *e)
{  ((OcDeviceGPUFull *)s->device)->eventsWaited++;
   OCH_CALL(och_stream_wait_event(((OcStreamGPU *)s)->handle, ((OcEventGPU *)e)->handle)); return 0;
}
static void OcFreeDeviceGPU(OcDevice *device)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device;
   och_device_set(device->index);
   while (g->freeStreams) { OcStream *s = g->freeStreams; g->freeStreams = s->next; och_stream_destroy(((OcStreamGPU *)s)->handle); OcFree(s); }
   while (g->freeEvents)  { OcEvent *e = g->freeEvents; g->freeEvents = e->next; och_event_destroy(((OcEventGPU *)e)->handle); OcFree(e); }
}
/* device_gpu.c:471-616: the properties under the reference's field names */
static void fill_public_properties(OcDevicePropGPU *q, const och_device_prop *p)
{  int i;
   memset(q, 0, sizeof(*q));
   memcpy(q->name, p->name, sizeof(q->name)); q->name[sizeof(q->name) - 1] = 0;
   q->totalGlobalMem = p->total_global_mem; q->freeGlobalMem = p->free_global_mem; q->sharedMemPerBlock = p->shared_mem_per_block;
   q->regsPerBlock = p->regs_per_block; q->warpSize = p->wavefront_size; q->memPitch = p->mem_pitch;
   q->maxThreadsPerBlock = p->max_threads_per_block;
   for (i = 0; i < 3; i++) { q->maxThreadsDim[i] = p->max_threads_dim[i]; q->maxGridSize[i] = p->max_grid_size[i]; }
   q->clockRate = p->clock_rate_khz; q->totalConstMem = p->total_const_mem; q->major = p->major; q->minor = p->minor;
   q->deviceOverlap = p->async_engine_count > 0; q->multiProcessorCount = p->multiprocessor_count;
   q->kernelExecTimeoutEnabled = p->kernel_exec_timeout_enabled; q->integrated = p->integrated;
   q->canMapHostMemory = p->can_map_host_memory; q->computeMode = p->compute_mode; q->concurrentKernels = p->concurrent_kernels;
   q->ECCEnabled = p->ecc_enabled; q->pciBusID = p->pci_bus_id; q->pciDeviceID = p->pci_device_id; q->pciDomainID = p->pci_domain_id;
   q->tccDriver = p->tcc_driver; q->asyncEngineCount = p->async_engine_count; q->unifiedAddressing = 1;
   q->memoryClockRate = p->memory_clock_rate_khz; q->memoryBusWidth = p->memory_bus_width; q->l2CacheSize = p->l2_cache_size;
   q->maxThreadsPerMultiProcessor = p->max_threads_per_multiprocessor;
   q->sharedMemPerMultiprocessor = p->shared_mem_per_block; q->maxSharedMemPerSM = (int)p->shared_mem_per_block;
   q->maxWarpsPerMultiProcessor = p->wavefront_size > 0 ? p->max_threads_per_multiprocessor / p->wavefront_size : 0;
}
/* device_gpu.c:81-122. A GPU device has NO default stream: every storage gets a stream of its own (storage.c:94-103),
   so that operations on different tensors overlap and are ordered by the read / write protocol only. */
static OcDevice *OcCreateDeviceGPU(OcDeviceType *type, int index, const char *name)
{  OcDevice *device = OcCreateDevice(type, index, name, sizeof(OcDeviceGPUFull)); OcDeviceGPUFull *g = (OcDeviceGPUFull *)device;
   if (device == NULL) return NULL;
   device->finalize = OcFreeDeviceGPU; device->endianness = 0; device->requiresAlignedData = 1;
   device->create_stream = OcDeviceGPU_createStream; device->create_event = OcDeviceGPU_createEvent;
   device->delete_stream = OcDeviceGPU_deleteStream; device->delete_event = OcDeviceGPU_deleteEvent;
   device->sync_stream = OcStreamGPU_synchronize;    device->sync_event = OcEventGPU_synchronize;
   device->record_event = OcEventGPU_record;          device->wait_event = OcStreamGPU_waitEvent;
   g->freeStreams = NULL; g->nFreeStreams = 0; g->freeEvents = NULL; g->nFreeEvents = 0;
   g->eventsRecorded = g->eventsWaited = g->streamsCreated = 0;
   if (och_device_properties(index, &g->hip) != 0 || och_device_warmup(index) != 0)                /* device_gpu.c:155-196, 471-616 */
   {  OcErrorMessage("%s", och_last_error()); OcDecrefDevice(device); return NULL; }
   fill_public_properties(&g->pub.properties, &g->hip);
   return device;
}

/* ---- storage (storage_gpu.c:61-302) ------------------------------------------------- */
static void OcStorageGPU_finalize(OcStorage *storage)
{  if (storage->data && OcStorage_isOwner(storage))
   {  och_device_set(storage->stream->device->index);
      och_free_async(storage->data, ((OcStreamGPU *)storage->stream)->handle);       /* stream-ordered: behind the storage's last work */
   }
}
static OcStorage *OcStorageGPU_create(OcSize nelem, OcDType dtype, OcDevice *device, OcStream *stream)
{  OcStorage *storage = OcAllocateStorage(device, dtype, stream, sizeof(OcStorageGPU)); void *ptr = NULL; OcSize size;
   if (storage == NULL) return NULL;
   storage->flags |= OC_STORAGE_OWNER; storage->finalize = OcStorageGPU_finalize; storage->data = NULL;
   size = nelem * storage->elemsize;
   storage->size = size; storage->capacity = size; storage->nelem = nelem;
   if (nelem > 0)
   {  if (activate(device) != 0) goto error;
      if (och_malloc_async(&ptr, (size_t)size, ((OcStreamGPU *)storage->stream)->handle) != 0)
      {  OcErrorMessage("Error allocating %s storage of size %lu on %s: %s", OcDType_name(dtype), (unsigned long)nelem, device->name, och_last_error());
         goto error;
      }
      storage->data = (char *)ptr;
   }
   return storage;
error:
   OcDecrefStorage(storage);
   return NULL;
}
int OcBufferGPU_copy(OcStorage *src, void *srcData, OcStorage *dst, void *dstData, OcDType dtype, OcSize n)
{  if (n == 0) return 0;
   if (src->stream->device != dst->stream->device) OcError(-1, "Copies between GPU devices are not part of this build (one device)");
   if (OcStorage_startRead(dst, src) != 0 || activate(dst->stream->device) != 0) return -1;
   OCH_CALL(och_memcpy_dtod_async(dstData, srcData, (size_t)(n * OcDType_size(dtype)), ((OcStreamGPU *)dst->stream)->handle));
   if (OcStorage_update(dst) != 0) return -1;
   return OcStorage_finishRead(dst, src);
}
/* the transfers between host and device block, as the reference's do (storage_gpu.c:165-250): wait for the storage's
   outstanding work, copy, record */
int OcBufferGPU_copyFromCPU(OcStorage *src, void *srcData, OcStorage *dst, void *dstData, OcDType dtype, OcSize n)
{  (void)src;
   if (OcStorage_synchronize(dst) != 0 || activate(dst->stream->device) != 0) return -1;
   OCH_CALL(och_memcpy_htod(dstData, srcData, (size_t)(n * OcDType_size(dtype)), ((OcStreamGPU *)dst->stream)->handle));
   return OcStorage_update(dst);
}
int OcBufferGPU_copyToCPU(OcStorage *src, void *srcData, OcStorage *dst, void *dstData, OcDType dtype, OcSize n)
{  if (OcStorage_synchronize(src) != 0 || activate(src->stream->device) != 0) return -1;
   OCH_CALL(och_memcpy_dtoh(dstData, srcData, (size_t)(n * OcDType_size(dtype)), ((OcStreamGPU *)src->stream)->handle));
   if (OcStorage_update(dst) != 0) return -1;
   return OcStorage_finishRead(src, src);                              /* updates the read event */
}
int OcBufferGPU_copyHostToStorage(OcStorage *storage, OcIndex offset, OcSize nbytes, void *ptr)
{  if (OcStorage_synchronize(storage) != 0 || activate(storage->stream->device) != 0) return -1;
   OCH_CALL(och_memcpy_htod(storage->data + offset, ptr, (size_t)nbytes, ((OcStreamGPU *)storage->stream)->handle));
   return OcStorage_update(storage);
}
int OcBufferGPU_copyStorageToHost(OcStorage *storage, OcIndex offset, OcSize nbytes, void *ptr)
{  if (OcStorage_synchronize(storage) != 0 || activate(storage->stream->device) != 0) return -1;
   OCH_CALL(och_memcpy_dtoh(ptr, storage->data + offset, (size_t)nbytes, ((OcStreamGPU *)storage->stream)->handle));
   return OcStorage_finishRead(storage, storage);
}
int OcBufferGPU_zero(OcStorage *storage, void *data, OcDType dtype, OcSize size)
{  if (activate(storage->stream->device) != 0) return -1;
   OCH_CALL(och_memset_async(data, 0, (size_t)(size * OcDType_size(dtype)), ((OcStreamGPU *)storage->stream)->handle));
   return OcStorage_update(storage);
}
static int OcDeviceGPU_formatInfo(OcDevice *device, char **str, const char *header, const char *footer)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device; size_t n = 512 + (header ? strlen(header) : 0) + (footer ? strlen(footer) : 0);
   if ((*str = (char *)OcMalloc(n)) == NULL) OcError(-1, "Insufficient memory for the device description");
   snprintf(*str, n, "%sDevice %s: %s (%s), %d compute units, %.1f GiB%s", header ? header : "", device->name, g->hip.name,
            g->hip.arch, g->hip.multiprocessor_count, g->hip.total_global_mem / 1073741824.0, footer ? footer : "");
   return 0;
}

/* ---- helpers for the glue ------------------------------------------------------------ */
static void scalar_value(const OcScalar *s, och_scalar *v) { memset(v, 0, sizeof(*v)); memcpy(v, &s->value, sizeof(*v) < sizeof(s->value) ? sizeof(*v) : sizeof(s->value)); }
static int same_shape(OcTensor *a, OcTensor *b)
{  int i; if (a->ndims != b->ndims) return 0;
   for (i = 0; i < a->ndims; i++) if (a->size[i] != b->size[i]) return 0;
   return 1;
}
#define SZ(t) ((const size_t *)(t)->size)

/* ---- copy ------------------------------------------------------------------------------ */
static int OcTensorGPU_copy(OcTensor *src, OcTensor *dst)
{  /* the swapping copy reverses the bytes of the SOURCE elements and then converts; a destination kept in the
      other byte order is swapped in place after a converting copy (src/core/cpu/op/tensor_copy_cpu.c:140-156) */
   int differ = (src->dtype != dst->dtype);
   int swap = differ ? OcTensor_isByteswapped(src) : (OcTensor_isByteswapped(src) != OcTensor_isByteswapped(dst));
   if (src->device != dst->device) OcError(-1, "Copies between GPU devices are not part of this build (one device)");
   if (src->nelem != dst->nelem) OcError(-1, "Mismatch in the number of elements in tensor copy");
   if (dst->nelem == 0) return 0;
   if (activate(dst->device) != 0 || OcTensor_startRead(dst, src) != 0) return -1;
   OCH_CALL((swap ? och_byteswap_copy : och_copy)(src->dtype, dst->dtype, src->ndims, SZ(src), src->strides, OcTensor_data(src),
                                                    dst->ndims, SZ(dst), dst->strides, OcTensor_data(dst), GPU_STREAM(dst)));
   if (differ && OcTensor_isByteswapped(dst))
      OCH_CALL(och_byteswap(dst->dtype, dst->ndims, SZ(dst), dst->strides, OcTensor_data(dst), GPU_STREAM(dst)));
   if (OcTensor_update(dst) != 0) return -1;
   return OcTensor_finishRead(dst, src);
}
/* Host tensors enter the device as the raw bytes of their memory extent and are converted, re-strided and byte-swapped
   there. The extent follows Ocean's convention (shape.c:82-125, used by tensor_copy_gpu.c:141-153): `offset` is the
   number of bytes in FRONT of the data pointer (negative strides), so the window starts at data - offset. */
static int OcTensorGPU_copyFromCPU(OcTensor *src, OcTensor *dst)
{  OcStorage *stage; OcTensor *view; OcSize offset, extent; int result;
   if (src->nelem != dst->nelem) OcError(-1, "Mismatch in the number of elements in tensor copy");
   if (dst->nelem == 0) return 0;
   if (OcShape_extent(src->ndims, src->size, src->strides, src->elemsize, &offset, &extent) != 0) return -1;
   if ((stage = OcStorage_createTemporary(extent, OcDTypeInt8, dst->device)) == NULL) return -1;
   if (OcBufferGPU_copyFromCPU(src->storage, OcTensor_data(src) - offset, stage, stage->data, OcDTypeInt8, extent) != 0)
   {  OcDecrefStorage(stage); return -1; }
   view = OcTensor_createFromStorage(stage, src->ndims, src->size, src->strides, offset, src->dtype);
   OcDecrefStorage(stage);
   if (view == NULL) return -1;
   OcTensor_setByteswapped(view, OcTensor_isByteswapped(src));
   result = OcTensorGPU_copy(view, dst);
   OcDecrefTensor(view);
   return result;
}
static int OcTensorGPU_copyToCPU(OcTensor *src, OcTensor *dst)
{  OcTensor *dense; int result; OcSize i, n = src->nelem; int es = dst->elemsize;
   char *host;
   if (src->nelem != dst->nelem) OcError(-1, "Mismatch in the number of elements in tensor copy");
   if (n == 0) return 0;
   /* convert / gather on the device into a dense tensor of the destination's type and byte order */
   if ((dense = OcTensor_createTemporary(dst->ndims, dst->size, NULL, dst->dtype, src->device)) == NULL) return -1;
   OcTensor_setByteswapped(dense, OcTensor_isByteswapped(dst));
   result = OcTensorGPU_copy(src, dense);
   if (result == 0 && OcTensor_isContiguous(dst))
      result = OcBufferGPU_copyToCPU(dense->storage, OcTensor_data(dense), dst->storage, OcTensor_data(dst), dst->dtype, n);
   else if (result == 0)
   {  /* strided host destination: download densely, then place element by element */
      if ((host = (char *)OcMalloc((size_t)(n * es))) == NULL) { OcErrorMessage("Insufficient memory for the host staging buffer"); result = -1; }
      else
      {  result = OcBufferGPU_copyToCPU(dense->storage, OcTensor_data(dense), dst->storage, host, dst->dtype, n);
         if (result == 0)
         {  OcSize idx[OC_TENSOR_MAX_DIMS] = { 0 }; int d;
            for (i = 0; i < n; i++)
            {  OcIndex off = 0;
               for (d = 0; d < dst->ndims; d++) off += idx[d] * dst->strides[d];
               memcpy(OcTensor_data(dst) + off, host + i * es, (size_t)es);
               for (d = 0; d < dst->ndims; d++) { if (++idx[d] < dst->size[d]) break; idx[d] = 0; }
            }
         }
         OcFree(host);
      }
   }
   OcDecrefTensor(dense);
   return result;
}
static int OcTensorGPU_byteswapNoFlag(OcTensor *tensor)
{  if (tensor->nelem == 0) return 0;
   if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_byteswap(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}

/* ---- fill / steps ------------------------------------------------------------------------ */
static int OcTensorGPU_fill(OcTensor *tensor, OcScalar *scalar)
{  och_scalar v; scalar_value(scalar, &v);
   if (scalar->dtype != tensor->dtype) OcError(-1, "Fill value must have the tensor's data type");
   if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_fill(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), v, GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}
static int OcTensorGPU_fillNaN(OcTensor *tensor, OcScalar *scalar)
{  och_scalar v; scalar_value(scalar, &v);
   if (!OcDType_isFloat(tensor->dtype)) return 0;                                    /* integers hold no NaN: nothing to do */
   if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_fill_nan(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), v, GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}
static int OcTensorGPU_maskedFill(OcTensor *tensor, OcTensor *mask, OcScalar *scalar)
{  och_scalar v; scalar_value(scalar, &v);
   if (mask->dtype != OcDTypeBool || !same_shape(tensor, mask)) OcError(-1, "Masked fill needs a Boolean mask of the tensor's shape");
   if (activate(tensor->device) != 0 || OcTensor_startRead(tensor, mask) != 0) return -1;
   OCH_CALL(och_masked_fill(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), mask->strides, OcTensor_data(mask), v, GPU_STREAM(tensor)));
   if (OcTensor_update(tensor) != 0) return -1;
   return OcTensor_finishRead(tensor, mask);
}
static int OcTensorGPU_stepsInt64(OcTensor *tensor, OcInt64 offset, OcInt64 step)
{  if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_steps_int64(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), offset, step, GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}
static int OcTensorGPU_stepsDouble(OcTensor *tensor, OcDouble offset, OcDouble step)
{  if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_steps_double(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), offset, step, GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}
static int OcTensorGPU_stepsCDouble(OcTensor *tensor, OcCDouble offset, OcCDouble step)
{  och_cdouble o, s; o.real = offset.real; o.imag = offset.imag; s.real = step.real; s.imag = step.imag;
   if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_steps_cdouble(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), o, s, GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}

/* ---- index operations (op/tensor_index_gpu.c:58-265) -------------------------------------- */
static int OcTensorGPU_addIfNegative(OcTensor *tensor, OcScalar *scalar)
{  och_scalar v; scalar_value(scalar, &v);
   if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_add_if_negative(tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), v, GPU_STREAM(tensor)));
   return OcTensor_update(tensor);
}
/* tensor: nstrides x nelem indices; offsets: nelem int64 values */
static int OcTensorGPU_indexToOffset(OcTensor *tensor, OcInt64 *strides, OcTensor *offsets)
{  OcIndex stride1, strideReduce; OcSize nelem; int nstrides;
   if (offsets->dtype != OcDTypeInt64) OcError(-1, "Offsets must be int64");
   if (tensor->ndims == 1) { stride1 = tensor->strides[0]; strideReduce = 0; nstrides = 1; nelem = tensor->size[0]; }      /* one index per element */
   else { stride1 = tensor->strides[1]; strideReduce = tensor->strides[0]; nstrides = (int)tensor->size[0]; nelem = tensor->size[1]; }
   if (activate(tensor->device) != 0 || OcTensor_startRead(offsets, tensor) != 0) return -1;
   OCH_CALL(och_index_to_offset(tensor->dtype, nstrides, (const int64_t *)strides, strideReduce, (size_t)nelem, stride1, OcTensor_data(tensor),
                                offsets->strides[0], OcTensor_data(offsets), GPU_STREAM(offsets)));
   if (OcTensor_update(offsets) != 0) return -1;
   return OcTensor_finishRead(offsets, tensor);
}
static int index_tables(OcTensorIndexView *view, int64_t **tables)
{  int d;
   for (d = 0; d < view->ndims; d++) tables[d] = (view->offsets && view->offsets[d]) ? (int64_t *)OcTensor_data(view->offsets[d]) : NULL;
   return 0;
}
/* the offset tables are tensors with storages (and streams) of their own, written by indexToOffset: the launch is
   ordered behind their writers and they are released to later writers afterwards (tensor_index_gpu.c:155-172, 199-216, 248-260) */
static int index_start(OcTensorIndexView *view, OcTensor *target)
{  int d;
   for (d = 0; d < view->ndims; d++) if (view->offsets && view->offsets[d] && OcTensor_startRead(target, view->offsets[d]) != 0) return -1;
   return 0;
}
static int index_finish(OcTensorIndexView *view, OcTensor *target)
{  int d;
   for (d = 0; d < view->ndims; d++) if (view->offsets && view->offsets[d] && OcTensor_finishRead(target, view->offsets[d]) != 0) return -1;
   return 0;
}
static int OcTensorGPU_getIndex(OcTensorIndexView *view, OcTensor *dst)
{  int64_t *tables[OC_TENSOR_MAX_DIMS]; OcTensor *v = view->view;
   index_tables(view, tables);
   if (activate(dst->device) != 0 || OcTensor_startRead(dst, v) != 0 || index_start(view, dst) != 0) return -1;
   OCH_CALL(och_get_index(v->dtype, view->ndims, SZ(v), tables, v->strides, OcTensor_data(v), dst->strides, OcTensor_data(dst), GPU_STREAM(dst)));
   if (OcTensor_update(dst) != 0 || OcTensor_finishRead(dst, v) != 0) return -1;
   return index_finish(view, dst);
}
static int OcTensorGPU_setIndex(OcTensorIndexView *view, OcTensor *src)
{  int64_t *tables[OC_TENSOR_MAX_DIMS]; OcTensor *v = view->view;
   index_tables(view, tables);
   if (activate(v->device) != 0 || OcTensor_startRead(v, src) != 0 || index_start(view, v) != 0) return -1;
   OCH_CALL(och_set_index(v->dtype, view->ndims, SZ(v), tables, v->strides, OcTensor_data(v), src->strides, OcTensor_data(src), GPU_STREAM(v)));
   if (OcTensor_update(v) != 0 || OcTensor_finishRead(v, src) != 0) return -1;
   return index_finish(view, v);
}
static int OcTensorGPU_fillIndex(OcTensorIndexView *view, OcScalar *scalar)
{  int64_t *tables[OC_TENSOR_MAX_DIMS]; OcTensor *v = view->view; och_scalar val; scalar_value(scalar, &val);
   index_tables(view, tables);
   if (activate(v->device) != 0 || index_start(view, v) != 0) return -1;
   OCH_CALL(och_fill_index(v->dtype, view->ndims, SZ(v), tables, v->strides, OcTensor_data(v), val, GPU_STREAM(v)));
   if (OcTensor_update(v) != 0) return -1;
   return index_finish(view, v);
}

/* Positions of the non-zero elements of a bool tensor (the reference implements these on the CPU only,
   src/core/cpu/op/tensor_index_cpu.c:60-155; its GPU table leaves the two entries empty). The result lives on
   the tensor's device: find -> int64 tensor of size ndims x nnz, maskToOffset -> nnz offsets sum(index * stride). */
static OcTensor *find_common(OcTensor *tensor, OcIndex *multiplier)
{  OcStorage *work; OcTensor *result = NULL; size_t nnz = 0; OcSize rsize[2]; int64_t mult[OC_TENSOR_MAX_DIMS]; int i;
   if (tensor->dtype != OcDTypeBool) { OcErrorMessage("Find requires a Boolean tensor"); return NULL; }
   if (activate(tensor->device) != 0) return NULL;
   /* the counts are produced and read on the tensor's stream */
   work = OcStorage_createWithStream((OcSize)och_find_workspace_size((size_t)tensor->nelem), OcDTypeInt8, tensor->storage->stream);
   if (work == NULL) return NULL;
   if (och_find_count(tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), work->data, &nnz, GPU_STREAM(tensor)) != 0)
   {  OcErrorMessage("%s", och_last_error()); goto final; }
   if (OcStorage_update(work) != 0) goto final;
   if (multiplier) { rsize[0] = (OcSize)nnz; result = OcTensor_create(1, rsize, NULL, OcDTypeInt64, tensor->device); }
   else { rsize[0] = tensor->ndims; rsize[1] = (OcSize)nnz; result = OcTensor_create(2, rsize, NULL, OcDTypeInt64, tensor->device); }
   if (result == NULL) goto final;
   for (i = 0; multiplier && i < tensor->ndims; i++) mult[i] = multiplier[i];
   if (OcTensor_startRead(result, tensor) != 0 || OcStorage_startRead(result->storage, work) != 0) { OcDecrefTensor(result); result = NULL; goto final; }
   if (och_find_apply(tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor), work->data, multiplier ? mult : NULL,
                      (int64_t *)OcTensor_data(result), GPU_STREAM(result)) != 0)
   {  OcErrorMessage("%s", och_last_error()); OcDecrefTensor(result); result = NULL; goto final; }
   if (OcTensor_update(result) != 0 || OcTensor_finishRead(result, tensor) != 0 || OcStorage_finishRead(result->storage, work) != 0)
   {  OcDecrefTensor(result); result = NULL; }
final:
   OcDecrefStorage(work);
   return result;
}
static OcTensor *OcTensorGPU_find(OcTensor *tensor) { return find_common(tensor, NULL); }
static OcTensor *OcTensorGPU_maskToOffset(OcTensor *tensor, OcIndex *strides) { return find_common(tensor, strides); }

/* ---- elementwise (op/tensor_unary_gpu.c:59-93, op/tensor_binary_gpu.c:58-97) ------------ */
static int unary_call(int op, const char *name, OcTensor *src, OcTensor *dst)
{  if (!och_unary_supported(op, src->dtype)) OcError(-1, "Function %s is not supported for type %s on GPU", name, OcDType_name(src->dtype));
   if ((int)dst->dtype != och_unary_result_dtype(op, src->dtype)) OcError(-1, "Invalid destination type in %s", name);
   if (!same_shape(src, dst)) OcError(-1, "Mismatch in tensor sizes in %s", name);
   if (activate(dst->device) != 0 || OcTensor_startRead(dst, src) != 0) return -1;
   OCH_CALL(och_unary(op, src->dtype, dst->ndims, SZ(dst), src->strides, OcTensor_data(src), dst->strides, OcTensor_data(dst), GPU_STREAM(dst)));
   if (OcTensor_update(dst) != 0) return -1;
   return OcTensor_finishRead(dst, src);
}
static int binary_call(int op, const char *name, OcTensor *src1, OcTensor *src2, OcTensor *dst)
{  if (!och_binary_supported(op, src1->dtype)) OcError(-1, "Function %s is not supported for type %s on GPU", name, OcDType_name(src1->dtype));
   if ((int)src2->dtype != och_binary_operand2_dtype(op, src1->dtype) || (int)dst->dtype != och_binary_result_dtype(op, src1->dtype))
      OcError(-1, "Invalid operand types in %s", name);
   if (!same_shape(src1, dst) || !same_shape(src2, dst)) OcError(-1, "Mismatch in tensor sizes in %s", name);
   if (activate(dst->device) != 0 || OcTensor_startRead(dst, src1) != 0 || OcTensor_startRead(dst, src2) != 0) return -1;
   OCH_CALL(och_binary(op, src1->dtype, dst->ndims, SZ(dst), src1->strides, OcTensor_data(src1), src2->strides, OcTensor_data(src2),
                       dst->strides, OcTensor_data(dst), GPU_STREAM(dst)));
   if (OcTensor_update(dst) != 0) return -1;
   if (OcTensor_finishRead(dst, src2) != 0) return -1;
   return OcTensor_finishRead(dst, src1);
}
#define OC_X(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *src, OcTensor *dst) { return unary_call(OP, #NAME, src, dst); }
OC_UNARY_TABLE(OC_X)
#undef OC_X
#define OC_X(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *a, OcTensor *b, OcTensor *c) { return binary_call(OP, #NAME, a, b, c); }
OC_BINARY_TABLE(OC_X)
#undef OC_X

/* ---- full reductions (op/tensor_reduce_all_gpu.c:201-444) --------------------------------- */
static int reduce_call(int op, OcTensor *tensor, OcScalar *lower, OcScalar *upper, double p, void *result)
{  och_scalar b1, b2;
   if (!och_reduce_supported(op, tensor->dtype)) OcError(-1, "Reduction is not supported for type %s on GPU", OcDType_name(tensor->dtype));
   if (OcTensor_isByteswapped(tensor)) OcError(-1, "Reductions need native byte order");
   if (lower) scalar_value(lower, &b1);
   if (upper) scalar_value(upper, &b2);
   if (activate(tensor->device) != 0) return -1;
   OCH_CALL(och_reduce_all(op, tensor->dtype, tensor->ndims, SZ(tensor), tensor->strides, OcTensor_data(tensor),
                           lower ? &b1 : NULL, upper ? &b2 : NULL, p, result, NULL, GPU_STREAM(tensor)));
   return 0;
}
#define OC_REDUCE_BOOL(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *t, int *result) \
   { unsigned char r = 0; if (reduce_call(OP, t, NULL, NULL, 0.0, &r) != 0) return -1; *result = r ? 1 : 0; return 0; }
OC_REDUCE_BOOL(any, OCH_R_ANY) OC_REDUCE_BOOL(all, OCH_R_ALL)
static int float_only(int op, OcTensor *t, int ifnot, int *result)
{  unsigned char r = 0;
   if (!OcDType_isFloat(t->dtype)) { *result = ifnot; return 0; }            /* integers are always finite */
   if (reduce_call(op, t, NULL, NULL, 0.0, &r) != 0) return -1;
   *result = r ? 1 : 0; return 0;
}
static int OcTensorGPU_allFinite(OcTensor *t, int *result) { return float_only(OCH_R_ALL_FINITE, t, 1, result); }
static int OcTensorGPU_anyInf(OcTensor *t, int *result)    { return float_only(OCH_R_ANY_INF, t, 0, result); }
static int OcTensorGPU_anyNaN(OcTensor *t, int *result)    { return float_only(OCH_R_ANY_NAN, t, 0, result); }
static int OcTensorGPU_nnz(OcTensor *t, OcUInt64 *result)    { return reduce_call(OCH_R_NNZ, t, NULL, NULL, 0.0, result); }
static int OcTensorGPU_nnzNaN(OcTensor *t, OcUInt64 *result) { return reduce_call(OCH_R_NNZ_NAN, t, NULL, NULL, 0.0, result); }
#define OC_REDUCE_RANGE2(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *t, OcScalar *lo, OcScalar *hi, int *result) \
   { unsigned char r = 0; if (reduce_call(OP, t, lo, hi, 0.0, &r) != 0) return -1; *result = r ? 1 : 0; return 0; }
#define OC_REDUCE_RANGE1(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *t, OcScalar *bound, int *result) \
   { unsigned char r = 0; if (reduce_call(OP, t, bound, NULL, 0.0, &r) != 0) return -1; *result = r ? 1 : 0; return 0; }
OC_REDUCE_RANGE2(allGELE, OCH_R_ALL_GELE) OC_REDUCE_RANGE2(allGELT, OCH_R_ALL_GELT) OC_REDUCE_RANGE2(allGTLE, OCH_R_ALL_GTLE) OC_REDUCE_RANGE2(allGTLT, OCH_R_ALL_GTLT)
OC_REDUCE_RANGE1(allLE, OCH_R_ALL_LE) OC_REDUCE_RANGE1(allLT, OCH_R_ALL_LT) OC_REDUCE_RANGE1(allGE, OCH_R_ALL_GE) OC_REDUCE_RANGE1(allGT, OCH_R_ALL_GT)
static int scalar_reduce(int op, OcTensor *t, double p, OcScalar *result)
{  memset(result, 0, sizeof(*result));
   if (reduce_call(op, t, NULL, NULL, p, &result->value) != 0) return -1;
   result->dtype = (OcDType)och_reduce_result_dtype(op, t->dtype);
   return 0;
}
#define OC_REDUCE_SCALAR(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *t, OcScalar *result) { return scalar_reduce(OP, t, 0.0, result); }
OC_REDUCE_SCALAR(sum, OCH_R_SUM) OC_REDUCE_SCALAR(prod, OCH_R_PROD) OC_REDUCE_SCALAR(sumNaN, OCH_R_SUM_NAN) OC_REDUCE_SCALAR(prodNaN, OCH_R_PROD_NAN)
OC_REDUCE_SCALAR(sumAbs, OCH_R_SUM_ABS) OC_REDUCE_SCALAR(sumAbsNaN, OCH_R_SUM_ABS_NAN) OC_REDUCE_SCALAR(maximum, OCH_R_MAXIMUM) OC_REDUCE_SCALAR(minimum, OCH_R_MINIMUM)
OC_REDUCE_SCALAR(maximumAbs, OCH_R_MAXIMUM_ABS) OC_REDUCE_SCALAR(minimumAbs, OCH_R_MINIMUM_ABS) OC_REDUCE_SCALAR(norm2, OCH_R_NORM2) OC_REDUCE_SCALAR(norm2NaN, OCH_R_NORM2_NAN)
static int OcTensorGPU_norm(OcTensor *t, double p, OcScalar *result)    { return scalar_reduce(OCH_R_NORM, t, p, result); }
static int OcTensorGPU_normNaN(OcTensor *t, double p, OcScalar *result) { return scalar_reduce(OCH_R_NORM_NAN, t, p, result); }

/* ---- axis reductions (op/tensor_reduce_axis_gpu.c:108-281) --------------------------------- */
static int axis_call(int op, OcTensor *src, double p, int n, int *axes, OcTensor *dst)
{  OcSolidReduceAxis a; och_reduce_axis_config c; int i;
   memset(&a, 0, sizeof(a));
   if (!och_reduce_supported(op, src->dtype)) OcError(-1, "Axis reduction is not supported for type %s on GPU", OcDType_name(src->dtype));
   if ((int)dst->dtype != och_reduce_result_dtype(op, src->dtype)) OcError(-1, "Invalid destination type in axis reduction");
   if (OcTensor_isByteswapped(src) || OcTensor_isByteswapped(dst)) OcError(-1, "Axis reductions need native byte order");
   if (dst->nelem == 0) return 0;
   OcSolid_analyzeReduceAxis(&a, src, dst, n, axes, 0);
   memset(&c, 0, sizeof(c));
   c.ndims = a.ndims; c.rdims = a.rdims;
   for (i = 0; i < a.ndims; i++) { c.size[i] = (size_t)a.size[i]; c.strides1[i] = a.strides1[i]; c.strides2[i] = a.strides2[i]; }
   for (i = 0; i < a.rdims; i++) { c.rsize[i] = (size_t)a.rsize[i]; c.rstrides[i] = a.rstrides[i]; }
   c.ptr1 = a.ptr1; c.ptr2 = a.ptr2; c.stream = GPU_STREAM(dst);
   if (activate(dst->device) != 0 || OcTensor_startRead(dst, src) != 0) return -1;
   OCH_CALL(och_reduce_axis(op, src->dtype, &c, p));
   if (OcTensor_update(dst) != 0) return -1;
   return OcTensor_finishRead(dst, src);
}
#define OC_X(NAME, OP) static int OcTensorGPU_##NAME(OcTensor *src, int n, int *axes, OcTensor *dst) { return axis_call(OP, src, 0.0, n, axes, dst); }
OC_AXIS_TABLE(OC_X)
#undef OC_X
static int OcTensorGPU_axisNorm(OcTensor *src, double p, int n, int *axes, OcTensor *dst)    { return axis_call(OCH_R_NORM, src, p, n, axes, dst); }
static int OcTensorGPU_axisNormNaN(OcTensor *src, double p, int n, int *axes, OcTensor *dst) { return axis_call(OCH_R_NORM_NAN, src, p, n, axes, dst); }

/* ---- GEMM (op/tensor_blas_gpu.c:63-286) ------------------------------------------------------ */
static int OcTensorGPU_gemm(OcSize M, OcSize N, OcSize K, char transA, char transB, OcTensor *alpha, OcTensor *A, OcIndex ldA,
                            OcTensor *B, OcIndex ldB, OcTensor *beta, OcTensor *C, OcIndex ldC)
{  OcIndex index[OC_TENSOR_MAX_DIMS] = { 0 }; int i, ndims = A->ndims, host = (alpha->device == OcCPU);
   char *pa = OcTensor_data(alpha), *pb = OcTensor_data(beta), *pA = OcTensor_data(A), *pB = OcTensor_data(B), *pC = OcTensor_data(C);
   if (C->nelem == 0) return 0;
   if (K == 0) { ldA = N; ldB = M; }
   if (!och_gemm_supported(A->dtype)) OcError(-1, "Unsupported data type in function gpu gemm (%s)", OcDType_name(A->dtype));
   if (activate(A->device) != 0) return -1;
   /* the reference loops over the dimensions beyond the second (tensor_blas_gpu.c:171-252); here they are one batched launch */
   {  size_t bsize[OC_TENSOR_MAX_DIMS]; ptrdiff_t sa[OC_TENSOR_MAX_DIMS], sb[OC_TENSOR_MAX_DIMS], sA[OC_TENSOR_MAX_DIMS], sB[OC_TENSOR_MAX_DIMS], sC[OC_TENSOR_MAX_DIMS];
      int nb = 0;
      for (i = 2; i < ndims; i++, nb++)
      {  bsize[nb] = (size_t)A->size[i];
         sa[nb] = (i < alpha->ndims) ? alpha->strides[i] : 0; sb[nb] = (i < beta->ndims) ? beta->strides[i] : 0;
         sA[nb] = A->strides[i]; sB[nb] = B->strides[i]; sC[nb] = C->strides[i];
      }
      (void)index;
      OCH_CALL(och_gemm_batched(A->dtype, transA, transB, (size_t)M, (size_t)N, (size_t)K, pa, pA, ldA > 0 ? ldA : 1, pB, ldB > 0 ? ldB : 1, pb, pC, ldC,
                                nb, bsize, sa, sA, sB, sb, sC, host, GPU_STREAM(C)));
   }
   return 0;
}
static int OcTensorGPU_gemmSupportedOn(OcDevice *device, OcDType dtype) { (void)device; return och_gemm_supported(dtype); }

/* ---- beside the table: fused Gram-Schmidt projection (no slot in OcModuleCore, no counterpart in the reference) -------- */
/* v <- v - sum_i q_i (q_i^H v), one column of Q after the other; Q is n x k with dense columns, v a dense vector of n
   elements, r NULL or a dense vector of k elements that receives the coefficients; all on the same GPU, same type */
int OcTensorGPU_projectColumns(OcTensor *Q, OcTensor *v, OcTensor *r)
{  OcSize n, k; OcIndex es;
   if (Q == NULL || v == NULL) OcError(-1, "projectColumns: missing operand");
   es = OcDType_size(Q->dtype);
   if (!OcDeviceGPU_isInstance(Q->device) || v->device != Q->device || (r && r->device != Q->device))
      OcError(-1, "projectColumns: all tensors must be on the same GPU device");
   if (v->dtype != Q->dtype || (r && r->dtype != Q->dtype)) OcError(-1, "projectColumns: mismatch in data types");
   if (Q->ndims < 1 || Q->ndims > 2 || v->ndims != 1) OcError(-1, "projectColumns: Q must be a matrix and v a vector");
   n = Q->size[0]; k = (Q->ndims == 2) ? Q->size[1] : 1;
   if (v->size[0] != n || (r && (r->ndims != 1 || r->size[0] != k))) OcError(-1, "projectColumns: mismatch in tensor sizes");
   if ((n > 1 && (Q->strides[0] != es || v->strides[0] != es)) || (r && k > 1 && r->strides[0] != es) ||
       (Q->ndims == 2 && k > 1 && (Q->strides[1] % es != 0 || Q->strides[1] < (OcIndex)(n * es))))
      OcError(-1, "projectColumns: columns and vectors must be dense");
   if (n == 0 || k == 0) return 0;
   if (activate(v->device) != 0 || OcTensor_startRead(v, Q) != 0) return -1;
   if (r && OcTensor_startRead(v, r) != 0) return -1;             /* r is written on v's stream: order it behind r's own work */
   OCH_CALL(och_mgs_project(Q->dtype, (size_t)n, (size_t)k, OcTensor_data(Q), (Q->ndims == 2 && k > 1) ? Q->strides[1] / es : (OcIndex)n,
                            OcTensor_data(v), r ? OcTensor_data(r) : NULL, GPU_STREAM(v)));
   if (OcTensor_update(v) != 0) return -1;
   if (r && OcTensor_finishRead(v, r) != 0) return -1;
   return OcTensor_finishRead(v, Q);
}

/* ---- module table and registration (module_core_gpu.c:40-145) ------------------------------------ */
static int initializeContext(OcDevice *device, OcDeviceModule *deviceModule, void **context)
{  OcModuleCoreGPU_Context *ctx;
   (void)deviceModule;
   /* assigned first, so that a partial initialisation is cleaned up by finalizeContext; the interface's part of the
      context holds the ring of temporary storages and the scalar slots (module_core.c:52-79) */
   *context = (void *)OcModuleCore_createContext(device, sizeof(OcModuleCoreGPU_Context));
   if ((ctx = (OcModuleCoreGPU_Context *)(*context)) == NULL) return -1;
   ctx->deviceIndex = device->index;
   return activate(device);
}
static void finalizeContext(OcDevice *device, OcDeviceModule *deviceModule, void *context)
{  (void)deviceModule;
   if (context == NULL) return;
   och_device_set(device->index); och_device_synchronize();        /* the temporaries may still be in use */
   OcModuleCore_freeContext((OcModuleCore_Context *)context);
}
static void finalizeModule(OcDeviceModule *deviceModule) { (void)deviceModule; }

/* The table is assembled from the same pieces as the reference's (module_core_gpu.c:40-63, tensor_gpu.c:35-50) */
int OcRegisterDevicesGPU(OcModuleCore *m) { m->Device_formatInfo = OcDeviceGPU_formatInfo; return 0; }
int OcRegisterStorageGPU(OcModuleCore *m)
{  m->Storage_create = OcStorageGPU_create; m->Storage_fromObject = NULL;
   m->Buffer_copy = OcBufferGPU_copy; m->Buffer_copyFromCPU = OcBufferGPU_copyFromCPU; m->Buffer_copyToCPU = OcBufferGPU_copyToCPU;
   m->Buffer_copyHostStorage = OcBufferGPU_copyHostToStorage; m->Buffer_copyStorageHost = OcBufferGPU_copyStorageToHost; m->Buffer_zero = OcBufferGPU_zero;
   return 0;
}
void OcTensorGPU_initializeCopyOps(OcModuleCore *m)
{  m->Tensor_copy = OcTensorGPU_copy; m->Tensor_copyFromCPU = OcTensorGPU_copyFromCPU; m->Tensor_copyToCPU = OcTensorGPU_copyToCPU;
   m->Tensor_byteswapNoFlag = OcTensorGPU_byteswapNoFlag;          /* CPU-only in the reference (template_byteswap.c:27-34) */
}
void OcTensorGPU_initializeFillOps(OcModuleCore *m)
{  m->Tensor_fill = OcTensorGPU_fill; m->Tensor_fillNaN = OcTensorGPU_fillNaN; m->Tensor_maskedFill = OcTensorGPU_maskedFill; }
void OcTensorGPU_initializeStepOps(OcModuleCore *m)
{  m->Tensor_stepsInt64 = OcTensorGPU_stepsInt64; m->Tensor_stepsDouble = OcTensorGPU_stepsDouble; m->Tensor_stepsCDouble = OcTensorGPU_stepsCDouble; }
void OcTensorGPU_initializeIndexOps(OcModuleCore *m)
{  m->Tensor_find = OcTensorGPU_find; m->Tensor_maskToOffset = OcTensorGPU_maskToOffset;   /* empty in the reference's GPU table (docs/future_work.md:33) */
   m->Tensor_indexToOffset = OcTensorGPU_indexToOffset; m->Tensor_addIfNegative = OcTensorGPU_addIfNegative;
   m->Tensor_getIndex = OcTensorGPU_getIndex; m->Tensor_setIndex = OcTensorGPU_setIndex; m->Tensor_fillIndex = OcTensorGPU_fillIndex;
}
#define OC_X(NAME, OP) m->Tensor_##NAME = OcTensorGPU_##NAME;
void OcTensorGPU_initializeUnaryOps(OcModuleCore *m)  { OC_UNARY_TABLE(OC_X) }
void OcTensorGPU_initializeBinaryOps(OcModuleCore *m) { OC_BINARY_TABLE(OC_X) }
void OcTensorGPU_initializeReduceAxisOps(OcModuleCore *m)
{  OC_AXIS_TABLE(OC_X)
   m->Tensor_axisNorm = OcTensorGPU_axisNorm; m->Tensor_axisNormNaN = OcTensorGPU_axisNormNaN;
}
#undef OC_X
void OcTensorGPU_initializeBlasOps(OcModuleCore *m) { m->Tensor_gemm = OcTensorGPU_gemm; m->Tensor_gemmSupportedOn = OcTensorGPU_gemmSupportedOn; }
void OcTensorGPU_initializeReduceAllOps(OcModuleCore *m)
{  m->Tensor_allGELE = OcTensorGPU_allGELE; m->Tensor_allGELT = OcTensorGPU_allGELT; m->Tensor_allGTLE = OcTensorGPU_allGTLE; m->Tensor_allGTLT = OcTensorGPU_allGTLT;
   m->Tensor_allLE = OcTensorGPU_allLE; m->Tensor_allLT = OcTensorGPU_allLT; m->Tensor_allGE = OcTensorGPU_allGE; m->Tensor_allGT = OcTensorGPU_allGT;
   m->Tensor_any = OcTensorGPU_any; m->Tensor_all = OcTensorGPU_all; m->Tensor_allFinite = OcTensorGPU_allFinite; m->Tensor_anyInf = OcTensorGPU_anyInf;
   m->Tensor_anyNaN = OcTensorGPU_anyNaN; m->Tensor_nnz = OcTensorGPU_nnz; m->Tensor_nnzNaN = OcTensorGPU_nnzNaN;
   m->Tensor_sum = OcTensorGPU_sum; m->Tensor_prod = OcTensorGPU_prod; m->Tensor_sumNaN = OcTensorGPU_sumNaN; m->Tensor_prodNaN = OcTensorGPU_prodNaN;
   m->Tensor_sumAbs = OcTensorGPU_sumAbs; m->Tensor_sumAbsNaN = OcTensorGPU_sumAbsNaN; m->Tensor_maximum = OcTensorGPU_maximum; m->Tensor_minimum = OcTensorGPU_minimum;
   m->Tensor_maximumAbs = OcTensorGPU_maximumAbs; m->Tensor_minimumAbs = OcTensorGPU_minimumAbs; m->Tensor_norm2 = OcTensorGPU_norm2; m->Tensor_norm2NaN = OcTensorGPU_norm2NaN;
   m->Tensor_norm = OcTensorGPU_norm; m->Tensor_normNaN = OcTensorGPU_normNaN;
}
int OcRegisterTensorGPU(OcModuleCore *m)
{  OcTensorGPU_initializeCopyOps(m); OcTensorGPU_initializeFillOps(m); OcTensorGPU_initializeStepOps(m);
   OcTensorGPU_initializeIndexOps(m); OcTensorGPU_initializeUnaryOps(m); OcTensorGPU_initializeBinaryOps(m);
   OcTensorGPU_initializeBlasOps(m); OcTensorGPU_initializeReduceAllOps(m); OcTensorGPU_initializeReduceAxisOps(m);
   return 0;
}
static int initializeFunctions(OcModuleCore *m)
{  memset(m, 0, sizeof(*m));
   m->HEAD.module = &oc_module_core;               /* registration increments its reference count */
   m->HEAD.initializeContext = initializeContext; m->HEAD.finalizeContext = finalizeContext; m->HEAD.finalizeModule = finalizeModule;
   if (OcRegisterDevicesGPU(m) != 0 || OcRegisterStorageGPU(m) != 0 || OcRegisterTensorGPU(m) != 0) return -1;
   return 0;
}

int OcDeviceGPUCount(void) { return oc_gpu_count; }
OcDevice *OcDeviceGPUByIndex(int index) { return (index >= 0 && index < oc_gpu_count) ? OcGPU[index] : NULL; }
int OcDeviceGPU_isInstance(OcDevice *device) { return (device != NULL && oc_device_type_gpu != NULL && device->type == oc_device_type_gpu); }
int OcDeviceGPU_peerAccess(int device1, int device2)
{  int result = 0;
   if (device1 == device2) return 1;
   if (och_device_can_access_peer(device1, device2, &result) != 0) return 0;
   return result;
}
int OcDeviceGPU_properties(OcDevice *device, void *och_device_prop_out)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device; size_t total = 0;
   if (!OcDeviceGPU_isInstance(device) || och_device_prop_out == NULL) OcError(-1, "Device properties: not a GPU device");
   OCH_CALL(och_device_mem_info(device->index, &g->hip.free_global_mem, &total));
   g->pub.properties.freeGlobalMem = g->hip.free_global_mem;
   memcpy(och_device_prop_out, &g->hip, sizeof(g->hip));
   return 0;
}
/* device_gpu.c:620-637 */
int OcDeviceGPU_updateProperties(OcDeviceGPU *device)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device; size_t total = 0;
   if (!OcDeviceGPU_isInstance((OcDevice *)device)) OcError(-1, "Update properties: not a GPU device");
   if (och_device_mem_info(((OcDevice *)device)->index, &g->hip.free_global_mem, &total) != 0)
      OcError(-1, "Error getting memory info in update properties function: %s", och_last_error());
   device->properties.freeGlobalMem = g->hip.free_global_mem;
   return 0;
}
/* events recorded, stream waits issued and streams created on a GPU device since it was created (no counterpart in the
   reference): what a test needs to see that operands on different streams really go through the event protocol */
int OcDeviceGPU_activity(OcDevice *device, long *eventsRecorded, long *eventsWaited, long *streamsCreated)
{  OcDeviceGPUFull *g = (OcDeviceGPUFull *)device;
   if (!OcDeviceGPU_isInstance(device)) OcError(-1, "Device activity: not a GPU device");
   if (eventsRecorded) *eventsRecorded = g->eventsRecorded;
   if (eventsWaited) *eventsWaited = g->eventsWaited;
   if (streamsCreated) *streamsCreated = g->streamsCreated;
   return 0;
}

/* device_gpu.c:196-250 */
static void OcFinalizeDevicesGPU(void)
{  int i;
   if (oc_device_type_gpu) { OcDecrefDeviceType(oc_device_type_gpu); oc_device_type_gpu = NULL; }
   if (OcGPU != NULL)
   {  for (i = 0; i < oc_gpu_count; i++)
         if (OcGPU[i] != NULL) { och_device_set(i); och_device_synchronize(); OcDecrefDevice(OcGPU[i]); OcGPU[i] = NULL; }
      OcFree(OcGPU); OcGPU = NULL;
   }
   oc_gpu_count = 0;
}
int OcInitDevicesGPU(void)
{  OcDeviceType *type; OcDevice *device; char name[16]; int count = 0, index;
   if (och_device_count(&count) != 0) count = 0;
   if ((type = OcCreateDeviceType("GPU")) == NULL) return -1;
   oc_device_type_gpu = OcIncrefDeviceType(type);
   if (count > 0)
   {  if ((OcGPU = (OcDevice **)OcMalloc(sizeof(OcDevice *) * (size_t)count)) == NULL) OcError(-1, "Error allocating GPU device buffer");
      for (index = 0; index < count; index++) OcGPU[index] = NULL;
   }
   oc_gpu_count = count;
   for (index = 0; index < count; index++)
   {  snprintf(name, sizeof(name), "gpu%d", index);
      device = OcCreateDeviceGPU(type, index, name);
      if (device != NULL && OcRegisterDevice(device) == 0) OcGPU[index] = device;       /* the creation reference is the list's */
      else { if (device) OcDecrefDevice(device); OcFinalizeDevicesGPU(); return -1; }
   }
   return 0;
}
/* module_core_gpu.c:127-145 */
int OcInitModuleCore_GPU(void)
{  if (OcModuleCore_initialize() != 0) return -1;
   if (initializeFunctions(&oc_module_core_gpu) != 0) return -1;
   return OcRegisterModule("GPU", (OcDeviceModule *)&oc_module_core_gpu, sizeof(oc_module_core_gpu));
}
void OcFinalizeGPU(void)
{  if (!oc_gpu_initialized) return;
   oc_gpu_initialized = 0;
   OcFinalizeDevicesGPU();
}
/* ocean_gpu.c:38-58: the devices first, then the module (registration creates the module's context on every
   device of the type that exists, device_module.c:388-405) */
int OcInitGPU(void)
{  if (oc_gpu_initialized) return 0;
   if (OcInitDevicesGPU() != 0) return -1;
   if (OcInitModuleCore_GPU() != 0) { OcFinalizeDevicesGPU(); return -1; }
   oc_gpu_initialized = 1;
   return OcFinalizeAddHandler(OcFinalizeGPU, "Finalize Ocean GPU");
}
