/* Stand-in for the parts of Ocean's base library (libocean_base) and interface layer (libocean_core) that surround the
 * GPU device module, so that the module -- host/gpu_module.c, which calls these functions by the reference's names --
 * can be driven where Ocean's libraries are not present. This file defines what those libraries own and the module
 * does NOT: errors, data-type properties, device types and devices, module registration, module contexts, storages,
 * the stream synchronisation protocol, tensors, shape routines. Behaviour follows the reference:
 *   src/base/error.c, dtype.c:88-178, device.c:213-236,588-676, device_module.c:313-422, storage.c:36-222,
 *   tensor.c:237-272, shape.c:82-125,196-360; src/core/interface/module_core.c:52-110, storage_itf.c:39-160,
 *   tensor_itf.c:49-53; src/external/ocean-solid/ocean_solid.c:382-462.
 */
#include "ocean_base.h"
#include "core_interface.h"
#include <stdarg.h>
#include <string.h>

/* ---- errors -------------------------------------------------------------- */
static __thread char oc_error_buffer[1024];
static __thread const char *oc_error_file = NULL;
static __thread size_t oc_error_line = 0;

char       *OcError_getBuffer(void)     { return oc_error_buffer; }
size_t      OcError_getBufferSize(void) { return sizeof(oc_error_buffer); }
void        OcError_setSource(const char *file, size_t line) { oc_error_file = file; oc_error_line = line; }
const char *OcError_lastError(void)     { return oc_error_buffer; }
const char *OcError_lastMessage(void)   { return oc_error_buffer; }

/* ---- finalisation handlers (src/base/ocean.c: last added runs first) ----------- */
#define OC_MAX_FINALIZERS 16
static void (*oc_finalizers[OC_MAX_FINALIZERS])(void);
static int oc_nfinalizers = 0;
int OcFinalizeAddHandler(void (*funptr)(void), const char *desc)
{  (void)desc;
   if (oc_nfinalizers >= OC_MAX_FINALIZERS) OcError(-1, "Too many finalization handlers");
   oc_finalizers[oc_nfinalizers++] = funptr;
   return 0;
}
void OcFinalize(void)
{  while (oc_nfinalizers > 0) oc_finalizers[--oc_nfinalizers]();
}

/* ---- data types ---------------------------------------------------------- */
static const int oc_dtype_size[OC_DTYPE_COUNT + 1] = { 1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 4, 8, 16, 0 };
static const char *oc_dtype_name[OC_DTYPE_COUNT + 1] = { "bool", "uint8", "uint16", "uint32", "uint64", "int8", "int16", "int32", "int64",
   "half", "float", "double", "chalf", "cfloat", "cdouble", "none" };

int OcDType_size(OcDType d)      { return ((int)d >= 0 && d <= OcDTypeNone) ? oc_dtype_size[d] : 0; }
const char *OcDType_name(OcDType d) { return ((int)d >= 0 && d <= OcDTypeNone) ? oc_dtype_name[d] : "invalid"; }
int OcDType_isFloat(OcDType d)   { return d >= OcDTypeHalf && d <= OcDTypeCDouble; }
int OcDType_isComplex(OcDType d) { return d >= OcDTypeCHalf && d <= OcDTypeCDouble; }
int OcDType_isSigned(OcDType d)  { return d >= OcDTypeInt8 && d <= OcDTypeCDouble; }
OcDType OcDType_getBaseType(OcDType d) { return OcDType_isComplex(d) ? (OcDType)(d - 3) : d; }
static int base_size(OcDType d) { return OcDType_size(OcDType_getBaseType(d)); }

/* The type able to represent both arguments (dtype.c:88-178): equal types stay; bool yields to anything;
   unsigned pairs take the wider; signed with unsigned of at least its width widens to the next signed
   size (int64 with uint64: double); floating types absorb integers whose bits fit the significand
   (11, 24, 52), otherwise widen to float / double; complex follows its component type. */
OcDType OcDType_getCommonType(OcDType a, OcDType b)
{
   if (a < b) { OcDType t = a; a = b; b = t; }
   if (a == b) return a;
   if (a == OcDTypeNone) return b;
   if (a == OcDTypeBool) return a;
   if (!OcDType_isSigned(a)) return a;                         /* both unsigned (or bool): larger enumerator is wider */
   if (!OcDType_isFloat(a))
   {  int sb = OcDType_size(b);
      if (b == OcDTypeBool || OcDType_isSigned(b) || sb < OcDType_size(a)) return a;
      if (sb == 1) return OcDTypeInt16;
      if (sb == 2) return OcDTypeInt32;
      if (sb == 4) return OcDTypeInt64;
      return OcDTypeDouble;
   }
   {  int cplx = OcDType_isComplex(a);
      int bits = OcDType_size(b) * 8;
      int limit = (base_size(a) == 2) ? 11 : (base_size(a) == 4 ? 24 : 52);
      if (cplx && OcDType_isComplex(b)) return a;
      if (OcDType_isFloat(b))
      {  if (!cplx) return a;
         if (OcDType_size(b) <= base_size(a)) return a;
         return (b == OcDTypeFloat) ? OcDTypeCFloat : OcDTypeCDouble;
      }
      if (bits <= limit) return a;
      if (bits <= 24) return cplx ? OcDTypeCFloat : OcDTypeFloat;
      return cplx ? OcDTypeCDouble : OcDTypeDouble;
   }
}

/* ---- device types and devices (device.c) -------------------------------------- */
#define OC_MAX_DEVICE_TYPES 8
static OcDeviceType *oc_device_types[OC_MAX_DEVICE_TYPES];
static int oc_ndevice_types = 0;

static OcDeviceType oc_cpu_type = { (char *)"CPU", 1, NULL, 0, NULL, 0, 0 };
static OcDevice oc_cpu_device = { &oc_cpu_type, 0, (char *)"cpu", 0, 0, 1, NULL, 0, 0, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL };
OcDevice *OcCPU = &oc_cpu_device;

OcDeviceType *OcDeviceTypeByName(const char *name)
{  int i;
   for (i = 0; i < oc_ndevice_types; i++) if (strcmp(oc_device_types[i]->name, name) == 0) return oc_device_types[i];
   return NULL;
}
OcDeviceType *OcCreateDeviceType(const char *name)
{  OcDeviceType *t = OcDeviceTypeByName(name);
   if (t) return t;                                                /* device.c: an existing type of that name is returned */
   if (oc_ndevice_types >= OC_MAX_DEVICE_TYPES) OcError(NULL, "Too many device types");
   if ((t = (OcDeviceType *)calloc(1, sizeof(OcDeviceType))) == NULL) OcError(NULL, "Insufficient memory for the device type");
   t->name = strdup(name); t->refcount = 1;
   oc_device_types[oc_ndevice_types++] = t;
   return t;
}
OcDeviceType *OcIncrefDeviceType(OcDeviceType *t) { if (t) t->refcount++; return t; }
void OcDecrefDeviceType(OcDeviceType *t)
{  int i;
   if (t == NULL || t == &oc_cpu_type || --t->refcount > 0) return;
   for (i = 0; i < oc_ndevice_types; i++) if (oc_device_types[i] == t) { oc_device_types[i] = oc_device_types[--oc_ndevice_types]; break; }
   /* finalizeModule of every registered table (device_module.c: OcDeviceTypeFinalizeModules) */
   {  size_t off = 0;
      while (off + sizeof(size_t) <= t->lutSize)
      {  size_t size = *(size_t *)(t->lutBuffer + off);
         OcDeviceModule *m = (OcDeviceModule *)(t->lutBuffer + off + sizeof(size_t));
         if (m->finalizeModule) m->finalizeModule(m);
         off += sizeof(size_t) + size;
      }
   }
   free(t->lutBuffer); free(t->devices); free(t->name); free(t);
}
OcDevice *OcCreateDevice(OcDeviceType *type, int index, const char *name, size_t size)
{  OcDevice *d;
   if (size < sizeof(OcDevice)) OcError(NULL, "Invalid device structure size");
   if ((d = (OcDevice *)calloc(1, size)) == NULL) OcError(NULL, "Insufficient memory for the device object");
   d->type = OcIncrefDeviceType(type); d->index = index; d->name = strdup(name); d->refcount = 1;
   return d;
}
/* one context slot per module registered for the device's type, created by the module's initializeContext
   (device_module.c: OcDeviceInitializeModules) */
static int device_initialize_modules(OcDevice *d)
{  OcDeviceType *t = d->type; size_t off = 0, k = 0, n = 0;
   while (off + sizeof(size_t) <= t->lutSize) { n++; off += sizeof(size_t) + *(size_t *)(t->lutBuffer + off); }
   if (n > d->contextCapacity)
   {  void **buf = (void **)calloc(n, sizeof(void *));
      if (buf == NULL) OcError(-1, "Insufficient memory for the device contexts");
      if (d->contextBuffer) { memcpy(buf, d->contextBuffer, d->contextSize * sizeof(void *)); free(d->contextBuffer); }
      d->contextBuffer = buf; d->contextCapacity = n;
   }
   for (off = 0, k = 0; k < n; k++)
   {  size_t size = *(size_t *)(t->lutBuffer + off);
      OcDeviceModule *m = (OcDeviceModule *)(t->lutBuffer + off + sizeof(size_t));
      if (k >= d->contextSize)
      {  d->contextBuffer[k] = NULL; d->contextSize = k + 1;
         if (m->initializeContext && m->initializeContext(d, m, &d->contextBuffer[k]) != 0) return -1;
      }
      off += sizeof(size_t) + size;
   }
   return 0;
}
int OcRegisterDevice(OcDevice *d)
{  OcDeviceType *t = d->type; OcDevice **list;
   if ((list = (OcDevice **)realloc(t->devices, sizeof(OcDevice *) * (size_t)(t->deviceCount + 1))) == NULL) OcError(-1, "Insufficient memory for the device list");
   t->devices = list; list[t->deviceCount++] = d;
   return device_initialize_modules(d);
}
OcDevice *OcIncrefDevice(OcDevice *d) { if (d) d->refcount++; return d; }
void OcDecrefDevice(OcDevice *d)
{  OcDeviceType *t; size_t off = 0, k = 0; int i;
   if (d == NULL || d == OcCPU || --d->refcount > 0) return;
   t = d->type;
   for (k = 0; k < d->contextSize && off + sizeof(size_t) <= t->lutSize; k++)            /* OcDeviceFinalizeModules */
   {  size_t size = *(size_t *)(t->lutBuffer + off);
      OcDeviceModule *m = (OcDeviceModule *)(t->lutBuffer + off + sizeof(size_t));
      if (m->finalizeContext) m->finalizeContext(d, m, d->contextBuffer[k]);
      off += sizeof(size_t) + size;
   }
   if (d->defaultStream) OcDecrefStream(d->defaultStream);
   if (d->finalize) d->finalize(d);
   for (i = 0; i < t->deviceCount; i++) if (t->devices[i] == d) { t->devices[i] = t->devices[--t->deviceCount]; break; }
   free(d->contextBuffer); free(d->name);
   OcDecrefDeviceType(t);
   free(d);
}
OcStream *OcIncrefStream(OcStream *s) { if (s) s->refcount++; return s; }
void OcDecrefStream(OcStream *s)
{  if (s == NULL) return;
   if (--s->refcount == 0) { OcStream_synchronize(s); s->device->delete_stream(s); }
}
OcStream *OcDevice_createStream(OcDevice *d) { return d->create_stream ? d->create_stream(d) : NULL; }
int  OcStream_synchronize(OcStream *s) { return s->device->sync_stream ? s->device->sync_stream(s) : 0; }
int  OcStream_waitFor(OcStream *s, OcEvent *e) { if (e == NULL) return 0; return s->device->wait_event(s, e); }
int  OcDevice_createEvent(OcDevice *d, OcEvent **e) { if (d->create_event == 0) { *e = NULL; return 0; } return d->create_event(d, e); }
void OcDevice_freeEvent(OcDevice *d, OcEvent *e) { if (e) d->delete_event(d, e); }
int  OcEvent_synchronize(OcDevice *d, OcEvent *e) { if (e == NULL) return 0; return d->sync_event(e); }
int  OcEvent_record(OcEvent *e, OcStream *s) { if (e == NULL) return 0; return s->device->record_event(e, s); }

/* ---- module registration (device_module.c:313-422) ------------------------------- */
struct __OcModule { const char *name; };
OcModule oc_module_core = { "core" };
int OcModuleCore_initialize(void) { return 0; }

/* The table is COPIED into the device type's look-up buffer (the registering module may keep its own in static
   storage), preceded by its size; the size must match the interface's view of the table (device_module.c:330).
   Devices of that type which exist already get their context for the new module. */
int OcRegisterModule(const char *deviceType, OcDeviceModule *info, size_t size)
{  OcDeviceType *t = OcDeviceTypeByName(deviceType); size_t need; int i;
   if (t == NULL) OcError(-1, "Device type %s does not exist", deviceType);
   if (info->module == &oc_module_core && size != sizeof(OcModuleCore))
      OcError(-1, "Mismatch in device module size (%zu, expected %zu)", size, sizeof(OcModuleCore));
   need = t->lutSize + sizeof(size_t) + size;
   if (need > t->lutCapacity)
   {  char *buf = (char *)realloc(t->lutBuffer, need);
      if (buf == NULL) OcError(-1, "Insufficient memory for the module look-up table");
      t->lutBuffer = buf; t->lutCapacity = need;
   }
   memcpy(t->lutBuffer + t->lutSize, &size, sizeof(size_t));
   memcpy(t->lutBuffer + t->lutSize + sizeof(size_t), info, size);
   ((OcDeviceModule *)(t->lutBuffer + t->lutSize + sizeof(size_t)))->available = 1;
   t->lutSize = need;
   for (i = 0; i < t->deviceCount; i++) if (device_initialize_modules(t->devices[i]) != 0) return -1;
   return 0;
}
static int core_module_slot(OcDeviceType *t, OcModuleCore **table)
{  size_t off = 0; int k = 0;
   while (off + sizeof(size_t) <= t->lutSize)
   {  size_t size = *(size_t *)(t->lutBuffer + off);
      OcDeviceModule *m = (OcDeviceModule *)(t->lutBuffer + off + sizeof(size_t));
      if (m->module == &oc_module_core) { if (table) *table = (OcModuleCore *)m; return k; }
      off += sizeof(size_t) + size; k++;
   }
   return -1;
}
OcModuleCore *OcModuleCore_forDevice(OcDevice *device)
{  OcModuleCore *table = NULL;
   if (device == NULL || device == OcCPU || device->type == NULL) return NULL;
   return core_module_slot(device->type, &table) >= 0 ? table : NULL;
}
OcModuleCore_Context *OcModuleCore_getContext(OcDevice *device)
{  int k;
   if (device == NULL || device == OcCPU || device->type == NULL) return NULL;
   k = core_module_slot(device->type, NULL);
   return (k >= 0 && (size_t)k < device->contextSize) ? (OcModuleCore_Context *)device->contextBuffer[k] : NULL;
}
/* module_core.c:52-79: the context every device module embeds at the start of its own: a ring of three temporary
   storages and the scalar-tensor slots */
OcModuleCore_Context *OcModuleCore_createContext(OcDevice *device, size_t size)
{  OcModuleCore_Context *ctx; int i, j;
   if (size < sizeof(OcModuleCore_Context) || (ctx = (OcModuleCore_Context *)calloc(1, size)) == NULL)
      OcError(NULL, "Error allocating the core module context for device %s", device->name);
   ctx->scalarCount = 8;
   for (i = 0; i < OC_DTYPE_COUNT; i++) { ctx->scalarIndex[i] = 0; for (j = 0; j < ctx->scalarCount; j++) ctx->scalarList[i][j] = NULL; }
   ctx->bufferCount = 3; ctx->bufferIndex = 0; ctx->bufferMaxSize = 0;
   if ((ctx->bufferList = (OcStorage **)calloc((size_t)ctx->bufferCount, sizeof(OcStorage *))) == NULL)
   {  free(ctx); OcError(NULL, "Error initializing buffer storage for device %s", device->name); }
   return ctx;
}
void OcModuleCore_freeContext(OcModuleCore_Context *ctx)
{  int i, j;
   if (ctx == NULL) return;
   if (ctx->bufferList) { for (i = 0; i < ctx->bufferCount; i++) if (ctx->bufferList[i]) OcDecrefStorage(ctx->bufferList[i]); free(ctx->bufferList); }
   for (i = 0; i < OC_DTYPE_COUNT; i++) for (j = 0; j < ctx->scalarCount; j++) if (ctx->scalarList[i][j]) OcDecrefTensor(ctx->scalarList[i][j]);
   free(ctx);
}

/* ---- storage (storage.c:36-222) -------------------------------------------------- */
static void deallocate_storage(OcStorage *s)
{  OcStream *stream;
   if (s == NULL) return;
   if ((stream = s->stream) != NULL)
   {  OcEvent_synchronize(stream->device, s->event);
      OcDevice_freeEvent(stream->device, s->event);
      OcDecrefStream(stream);
   }
   free(s);
}
/* size: bytes of the (device-specific) storage structure. With a stream the storage shares it; without one the
   device creates a new stream, so that work on different storages can overlap (storage.c:94-103). */
OcStorage *OcAllocateStorage(OcDevice *device, OcDType dtype, OcStream *stream, OcSize size)
{  OcStorage *s;
   if (dtype == OcDTypeNone) OcError(NULL, "Invalid data type in storage allocation");
   if ((s = (OcStorage *)calloc(1, (size_t)size)) == NULL) OcError(NULL, "Insufficient memory to allocate the storage structure");
   s->dtype = dtype; s->elemsize = OcDType_size(dtype); s->refcount = 1;
   if (stream != NULL) s->stream = OcIncrefStream(stream);
   else if (device->create_stream && (s->stream = OcDevice_createStream(device)) == NULL) { free(s); return NULL; }
   if (OcDevice_createEvent(device, &s->event) != 0) { deallocate_storage(s); return NULL; }
   return s;
}
OcStorage *OcIncrefStorage(OcStorage *s) { if (s) s->refcount++; return s; }
void OcDecrefStorage(OcStorage *s)
{  if (s == NULL || --s->refcount > 0) return;
   if (s->stream) OcStream_synchronize(s->stream);        /* outstanding work must have finished before the memory goes away (storage.c:51-57) */
   if (s->finalize) s->finalize(s);
   deallocate_storage(s);
}
int OcStorage_isOwner(OcStorage *s) { return (s->flags & OC_STORAGE_OWNER) ? 1 : 0; }
int OcStorage_synchronize(OcStorage *s) { if (s->stream == NULL) return 0; return OcEvent_synchronize(s->stream->device, s->event); }
/* The protocol (storage.c:141-222). Every storage has one event. After an operation was scheduled on a storage's
   stream, update() records the event there. startRead(s, r): s's stream waits for r's event (r's last write or read);
   finishRead(s, r): r's stream waits for s's event (the operation that read r) and r's event is recorded again on r's
   stream, so that a later writer of r waits for this reader. Host storages have neither stream nor event. */
int OcStorage_update(OcStorage *s) { if (s->stream == NULL) return 0; return OcEvent_record(s->event, s->stream); }
int OcStorage_startRead(OcStorage *s, OcStorage *r)
{  if (s->stream == NULL) return r->stream ? OcEvent_synchronize(r->stream->device, r->event) : 0;
   return OcStream_waitFor(s->stream, r->event);
}
int OcStorage_finishRead(OcStorage *s, OcStorage *r)
{  if (r->stream == NULL) return 0;
   if (OcStream_waitFor(r->stream, s->event) != 0) return -1;
   return OcEvent_record(r->event, r->stream);
}
int OcStorage_startWrite(OcStorage *s, OcStorage *w)
{  if (s->stream == NULL) return w->stream ? OcEvent_synchronize(w->stream->device, w->event) : 0;
   return OcStream_waitFor(s->stream, w->event);
}
int OcStorage_finishWrite(OcStorage *s, OcStorage *w)
{  if (w->stream == NULL) return 0;
   if (OcStream_waitFor(w->stream, s->event) != 0) return -1;
   return OcStorage_update(w);
}

/* interface layer (storage_itf.c:39-160) */
static void cpu_storage_finalize(OcStorage *s) { if (s->flags & OC_STORAGE_OWNER) free(s->data); }
static OcStorage *cpu_storage_create(OcSize nelem, OcDType dtype)
{  OcStorage *s = OcAllocateStorage(OcCPU, dtype, NULL, sizeof(OcStorage));
   if (s == NULL) return NULL;
   s->nelem = nelem; s->size = s->capacity = nelem * s->elemsize;
   s->data = (char *)malloc(s->size > 0 ? (size_t)s->size : 1);
   s->flags = OC_STORAGE_OWNER; s->finalize = cpu_storage_finalize;
   if (s->data == NULL) { OcErrorMessage("Insufficient memory to allocate %td bytes", s->size); free(s); return NULL; }
   return s;
}
OcStorage *OcStorage_create(OcSize nelem, OcDType dtype, OcDevice *device)
{  OcModuleCore *m;
   if (nelem < 0) OcError(NULL, "Storage size cannot be negative");
   if (device == OcCPU) return cpu_storage_create(nelem, dtype);
   m = OcModuleCore_forDevice(device);
   if (m == NULL || m->Storage_create == NULL) OcError(NULL, "Storage creation is not supported on device %s", device ? device->name : "(null)");
   return m->Storage_create(nelem, dtype, device, device->defaultStream);      /* no default stream: a stream of its own */
}
OcStorage *OcStorage_createWithStream(OcSize nelem, OcDType dtype, OcStream *stream)
{  OcModuleCore *m; OcDevice *device;
   if (stream == NULL) OcError(NULL, "Storage creation with a stream needs a stream");
   device = stream->device;
   m = OcModuleCore_forDevice(device);
   if (m == NULL || m->Storage_create == NULL) OcError(NULL, "Storage creation is not supported on device %s", device->name);
   return m->Storage_create(nelem, dtype, device, stream);
}
/* storage_itf.c:61-121: temporaries come from a ring of three storages per device; a slot is reused when nobody else
   holds it and it is large enough, so that releasing a temporary does not wait for the device */
OcStorage *OcStorage_createTemporary(OcSize nelem, OcDType dtype, OcDevice *device)
{  OcModuleCore_Context *ctx = OcModuleCore_getContext(device); OcStorage *buffer; OcSize requested; int elemsize = OcDType_size(dtype), idx;
   if (nelem < 0) OcError(NULL, "Storage size cannot be negative");
   requested = nelem * elemsize;
   if (ctx == NULL || ctx->bufferList == NULL || ctx->bufferCount == 0 || (requested > ctx->bufferMaxSize && ctx->bufferMaxSize > 0))
      return OcStorage_create(nelem, dtype, device);
   idx = ctx->bufferIndex; ctx->bufferIndex = (idx + 1) % ctx->bufferCount;
   buffer = ctx->bufferList[idx];
   if (buffer != NULL && buffer->refcount == 1)
   {  if (buffer->capacity >= requested)
      {  buffer->dtype = dtype; buffer->size = requested; buffer->nelem = nelem; buffer->elemsize = elemsize;
         buffer->flags &= ~(OcStorageFlags)(OC_STORAGE_BYTESWAPPED | OC_STORAGE_READONLY | OC_STORAGE_RAW);
         return OcIncrefStorage(buffer);
      }
      OcDecrefStorage(buffer); ctx->bufferList[idx] = NULL;
   }
   if ((buffer = OcStorage_create(nelem, dtype, device)) == NULL) return NULL;
   if (ctx->bufferList[idx] == NULL) ctx->bufferList[idx] = OcIncrefStorage(buffer);
   else if (ctx->bufferList[idx]->capacity < buffer->capacity) { OcDecrefStorage(ctx->bufferList[idx]); ctx->bufferList[idx] = OcIncrefStorage(buffer); }
   return buffer;
}

/* ---- shapes (shape.c) --------------------------------------------------------------- */
/* shape.c:82-125: dataOffset = bytes in FRONT of the data pointer (the spans of the negative strides, a non-negative
   number), dataExtent = bytes from the lowest to one past the highest address touched */
int OcShape_extent(int ndims, OcSize *size, OcIndex *strides, OcSize elemsize, OcSize *dataOffset, OcSize *dataExtent)
{  OcSize extent = elemsize, offset = 0; int i;
   for (i = 0; i < ndims; i++)
   {  OcSize d = size[i]; OcIndex s = strides ? strides[i] : 0;
      if (d == 0) { offset = 0; extent = 0; break; }
      if (strides == NULL) { extent *= d; continue; }
      if (d > 1) { if (s < 0) { offset += -s * (d - 1); extent += -s * (d - 1); } else extent += s * (d - 1); }
   }
   if (dataOffset) *dataOffset = offset;
   if (dataExtent) *dataExtent = extent;
   return 0;
}
static void normalize_strides(int ndims, OcSize *size, OcIndex *strides, OcIndex *offset)
{  OcIndex o = 0; int i;
   for (i = 0; i < ndims; i++) if (strides[i] < 0) { o += (size[i] - 1) * strides[i]; strides[i] = -strides[i]; }
   *offset = o;
}
static void normalize_strides2(int ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2, OcIndex *offset1, OcIndex *offset2)
{  OcIndex o1 = 0, o2 = 0; int i;          /* shape.c:216-236: the sign of strides2 decides */
   for (i = 0; i < ndims; i++)
      if (strides2[i] < 0)
      {  o1 += (size[i] - 1) * strides1[i]; o2 += (size[i] - 1) * strides2[i];
         strides1[i] = -strides1[i]; strides2[i] = -strides2[i];
      }
   *offset1 = o1; *offset2 = o2;
}
void OcShape_sortStrides2(int ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2)
{  int i, j;                      /* insertion sort: ascending strides1, ties by strides2 (shape.c:262-289) */
   for (i = 1; i < ndims; i++)
      for (j = i; j > 0; j--)
      {  int before = (strides1[j - 1] < strides1[j]) || (strides1[j - 1] == strides1[j] && strides2[j - 1] <= strides2[j]);
         OcSize s; OcIndex r;
         if (before) break;
         s = size[j]; size[j] = size[j - 1]; size[j - 1] = s;
         r = strides1[j]; strides1[j] = strides1[j - 1]; strides1[j - 1] = r;
         r = strides2[j]; strides2[j] = strides2[j - 1]; strides2[j - 1] = r;
      }
}
void OcShape_mergeBlocks2(int *ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2)
{  int i, j = 0, n = *ndims;       /* fold dimension i into j when both operands step contiguously (shape.c:334-360) */
   if (n <= 0) return;
   for (i = 1; i < n; i++)
   {  if (strides1[i] == strides1[j] * size[j] && strides2[i] == strides2[j] * size[j]) size[j] *= size[i];
      else { j++; size[j] = size[i]; strides1[j] = strides1[i]; strides2[j] = strides2[i]; }
   }
   *ndims = j + 1;
}
/* ocean_solid.c:382-462: kept dimensions (with the destination's strides) and reduced dimensions of an axis reduction,
   unit dimensions dropped, negative strides flipped into the base pointers, sorted and merged; the pointers in the
   configuration already include the offsets. */
void OcSolid_analyzeReduceAxis(OcSolidReduceAxis *c, OcTensor *src, OcTensor *dst, int n, int *axes, int flagRemoveRepeats)
{  OcSize size[OC_TENSOR_MAX_DIMS], rsize[OC_TENSOR_MAX_DIMS]; OcIndex strides1[OC_TENSOR_MAX_DIMS], strides2[OC_TENSOR_MAX_DIMS], rstrides[OC_TENSOR_MAX_DIMS], dummy[OC_TENSOR_MAX_DIMS];
   OcIndex offset1 = 0, offset2 = 0, roffset = 0; short reduced[OC_TENSOR_MAX_DIMS] = { 0 };
   int i, j = 0, k = 0, keepdims = (src->ndims == dst->ndims);
   for (i = 0; i < n; i++) reduced[axes[i]] = 1;
   for (i = 0; i < src->ndims; i++)
   {  if (reduced[i]) { if (keepdims) k++; continue; }
      if (src->size[i] != 1) { size[j] = src->size[i]; strides1[j] = src->strides[i]; strides2[j] = dst->strides[k]; j++; }
      k++;
   }
   c->ndims = j;
   for (i = 0, j = 0; i < n; i++)
   {  int a = axes[i];
      if (src->size[a] != 1 && !(flagRemoveRepeats && src->strides[a] == 0)) { rsize[j] = src->size[a]; rstrides[j] = src->strides[a]; j++; }
   }
   c->rdims = j;
   normalize_strides2(c->ndims, size, strides1, strides2, &offset1, &offset2);
   OcShape_sortStrides2(c->ndims, size, strides1, strides2);
   OcShape_mergeBlocks2(&c->ndims, size, strides1, strides2);
   normalize_strides(c->rdims, rsize, rstrides, &roffset);
   for (i = 0; i < c->rdims; i++) dummy[i] = rstrides[i];
   OcShape_sortStrides2(c->rdims, rsize, rstrides, dummy);
   for (i = 0; i < c->rdims; i++) dummy[i] = rstrides[i];
   OcShape_mergeBlocks2(&c->rdims, rsize, rstrides, dummy);
   for (i = 0; i < c->ndims; i++) { c->size[i] = (size_t)size[i]; c->strides1[i] = strides1[i]; c->strides2[i] = strides2[i]; }
   for (i = 0; i < c->rdims; i++) { c->rsize[i] = (size_t)rsize[i]; c->rstrides[i] = rstrides[i]; }
   c->ptr1 = OcTensor_data(src) + offset1 + roffset;
   c->ptr2 = OcTensor_data(dst) + offset2;
}

/* ---- tensors (tensor.c, tensor_itf.c) ------------------------------------------------ */
/* tensor.c:237-272: blockOffset and blockExtent in the convention of OcShape_extent (offset = bytes in front of the data) */
static void tensor_update_extent(OcTensor *t)
{  int i;
   t->nelem = 1;
   for (i = 0; i < t->ndims; i++) t->nelem *= t->size[i];
   OcShape_extent(t->ndims, t->size, t->strides, t->elemsize, &t->blockOffset, &t->blockExtent);
}
int OcTensor_extent(OcTensor *t, OcSize *offset, OcSize *extent)
{  if (offset) *offset = t->blockOffset;
   if (extent) *extent = t->blockExtent;
   return 0;
}
static OcTensor *tensor_header(int ndims, const OcSize *size, const OcIndex *strides, OcDType dtype)
{  OcTensor *t; int i;
   if (ndims < 0 || ndims > OC_TENSOR_MAX_DIMS) OcError(NULL, "Invalid number of tensor dimensions (%d)", ndims);
   if ((t = (OcTensor *)calloc(1, sizeof(OcTensor))) == NULL) OcError(NULL, "Insufficient memory to allocate the tensor object");
   t->ndims = ndims; t->capacity = OC_TENSOR_MAX_DIMS;
   t->size = (OcSize *)calloc(OC_TENSOR_MAX_DIMS, sizeof(OcSize));
   t->strides = (OcIndex *)calloc(OC_TENSOR_MAX_DIMS, sizeof(OcIndex));
   t->dtype = dtype; t->elemsize = OcDType_size(dtype); t->refcount = 1;
   {  OcIndex acc = t->elemsize;
      for (i = 0; i < ndims; i++)
      {  t->size[i] = size[i];
         t->strides[i] = strides ? strides[i] : acc;             /* default: column-major (docs/design_choices.md:25-27) */
         acc *= size[i];
      }
   }
   tensor_update_extent(t);
   return t;
}
OcTensor *OcTensor_createFromStorage(OcStorage *storage, int ndims, OcSize *size, OcIndex *strides, OcIndex offset, OcDType dtype)
{  OcTensor *t = tensor_header(ndims, size, strides, dtype);
   if (t == NULL) return NULL;
   if (t->nelem > 0 && (offset - t->blockOffset < 0 || offset - t->blockOffset + t->blockExtent > storage->size))
   {  OcErrorMessage("Tensor extent exceeds the storage size"); free(t->size); free(t->strides); free(t); return NULL; }
   t->storage = OcIncrefStorage(storage); t->offset = offset;
   t->device = storage->stream ? storage->stream->device : OcCPU;
   if (storage->flags & OC_STORAGE_BYTESWAPPED) t->flags |= OC_TENSOR_BYTESWAPPED;
   return t;
}
static OcTensor *tensor_create(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcDevice *device, OcStream *stream, int temporary)
{  OcTensor *probe = tensor_header(ndims, size, strides, dtype), *t;
   OcStorage *s; OcSize bytes, offset, nelem;
   if (probe == NULL) return NULL;
   bytes = probe->blockExtent; offset = probe->blockOffset;
   free(probe->size); free(probe->strides); free(probe);
   nelem = (bytes + OcDType_size(dtype) - 1) / OcDType_size(dtype);
   s = stream ? OcStorage_createWithStream(nelem, dtype, stream) : (temporary ? OcStorage_createTemporary(nelem, dtype, device) : OcStorage_create(nelem, dtype, device));
   if (s == NULL) return NULL;
   t = OcTensor_createFromStorage(s, ndims, size, strides, offset, dtype);
   OcDecrefStorage(s);
   return t;
}
OcTensor *OcTensor_create(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcDevice *device)
{  return tensor_create(ndims, size, strides, dtype, device, NULL, 0); }
OcTensor *OcTensor_createTemporary(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcDevice *device)
{  return tensor_create(ndims, size, strides, dtype, device, NULL, 1); }
OcTensor *OcTensor_createWithStream(int ndims, OcSize *size, OcIndex *strides, OcDType dtype, OcStream *stream)
{  if (stream == NULL) OcError(NULL, "Tensor creation with a stream needs a stream");
   return tensor_create(ndims, size, strides, dtype, stream->device, stream, 0);
}
OcTensor *OcTensor_shallowCopy(OcTensor *x)
{  OcTensor *t = OcTensor_createFromStorage(x->storage, x->ndims, x->size, x->strides, x->offset, x->dtype);
   if (t) t->flags = x->flags;
   return t;
}
OcTensor *OcIncrefTensor(OcTensor *t) { if (t) t->refcount++; return t; }
void OcDecrefTensor(OcTensor *t)
{  if (t == NULL || --t->refcount > 0) return;
   OcDecrefStorage(t->storage);
   free(t->size); free(t->strides); free(t);
}
int  OcTensor_isByteswapped(OcTensor *t) { return (t->flags & OC_TENSOR_BYTESWAPPED) ? 1 : 0; }
void OcTensor_setByteswapped(OcTensor *t, int flag)
{  if (flag) t->flags |= OC_TENSOR_BYTESWAPPED; else t->flags &= ~(OcTensorFlags)OC_TENSOR_BYTESWAPPED; }
int OcTensor_isContiguous(OcTensor *t)
{  OcIndex acc = t->elemsize; int i;
   for (i = 0; i < t->ndims; i++) { if (t->size[i] != 1 && t->strides[i] != acc) return 0; acc *= t->size[i]; }
   return 1;
}

/* views used by the front end (core_interface.h) */
OcTensor *OcTensor_transpose(OcTensor *x)
{  OcTensor *t = OcTensor_shallowCopy(x);
   if (t == NULL) return NULL;
   if (t->ndims < 2) { if (t->ndims == 1) { t->ndims = 2; t->size[1] = t->size[0]; t->strides[1] = t->strides[0]; t->size[0] = 1; t->strides[0] = t->elemsize; } return t; }
   {  OcSize s = t->size[0]; OcIndex r = t->strides[0];
      t->size[0] = t->size[1]; t->strides[0] = t->strides[1]; t->size[1] = s; t->strides[1] = r;
   }
   return t;
}
OcTensor *OcTensor_slice(OcTensor *x, int axis, OcSize start, OcSize count, OcIndex step)
{  OcTensor *t;
   if (axis < 0 || axis >= x->ndims || step == 0 || start < 0 || count < 0 ||
       (count > 0 && (start >= x->size[axis] || start + (count - 1) * step < 0 || start + (count - 1) * step >= x->size[axis])))
      OcError(NULL, "Slice out of range");
   if ((t = OcTensor_shallowCopy(x)) == NULL) return NULL;
   t->offset += start * t->strides[axis];
   t->size[axis] = count; t->strides[axis] *= step;
   tensor_update_extent(t);
   return t;
}
OcTensor *OcTensor_broadcastTo(OcTensor *x, int ndims, const OcSize *size)
{  OcTensor *t; int i;
   if (ndims < x->ndims) OcError(NULL, "Cannot broadcast to fewer dimensions");
   for (i = 0; i < x->ndims; i++)
      if (x->size[i] != size[i] && x->size[i] != 1) OcError(NULL, "Tensor dimensions are not compatible for broadcasting");
   if ((t = OcTensor_shallowCopy(x)) == NULL) return NULL;
   for (i = 0; i < ndims; i++)
   {  if (i >= x->ndims || (x->size[i] == 1 && size[i] != 1)) t->strides[i] = 0;
      t->size[i] = size[i];
   }
   t->ndims = ndims;
   tensor_update_extent(t);
   return t;
}

/* ---- layout self-description --------------------------------------------------- */
const char *OcHost_abiLayout(void)
{  static char buf[16384]; size_t n = 0;
   n += snprintf(buf + n, sizeof(buf) - n, "{");
#define S(T)    n += snprintf(buf + n, sizeof(buf) - n, "%s\"sizeof(" #T ")\": %zu", n > 1 ? ", " : "", sizeof(T));
#define F(T, M) n += snprintf(buf + n, sizeof(buf) - n, ", \"" #T "." #M "\": %zu", offsetof(T, M));
#include "abi_layout_fields.h"
#undef S
#undef F
   snprintf(buf + n, sizeof(buf) - n, "}");
   return buf;
}
