/* Base objects of the host stand-in: error messages, data-type properties, the CPU device,
 * storages, tensors and views, and the stream synchronisation protocol. Behaviour follows the
 * reference's base library (src/base/error.c, dtype.c:88-178, storage.c:36-160, tensor.c,
 * device.c) as far as the GPU device module depends on it. */
#include "ocean_host.h"
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ---- errors -------------------------------------------------------------- */
static __thread char oc_error_buffer[1024];

int OcErrorMessage(const char *fmt, ...)
{  va_list ap;
   va_start(ap, fmt);
   vsnprintf(oc_error_buffer, sizeof(oc_error_buffer), fmt, ap);
   va_end(ap);
   return -1;
}
const char *OcError_lastMessage(void) { return oc_error_buffer; }

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

/* ---- the CPU device (host memory; no streams) ------------------------------- */
static OcDevice oc_cpu_device = { NULL, 0, (char *)"cpu", 0, 0, 1, NULL, 0, 0, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL };
OcDevice *OcCPU = &oc_cpu_device;

/* ---- storage ------------------------------------------------------------------ */
static void cpu_storage_finalize(OcStorage *storage) { if (storage->flags & OC_STORAGE_OWNER) free(storage->data); }

OcStorage *OcStorage_create(OcSize nelem, OcDType dtype, OcDevice *device)
{
   if (device != OcCPU)
   {  OcModuleCore *m = OcModuleCore_forDevice(device);
      if (m == NULL || m->Storage_create == NULL) { OcErrorMessage("No storage support for device %s", device ? device->name : "(null)"); return NULL; }
      return m->Storage_create(nelem, dtype, device, device->defaultStream);
   }
   OcStorage *s = (OcStorage *)calloc(1, sizeof(OcStorage));
   if (s == NULL) { OcErrorMessage("Insufficient memory to allocate the storage object"); return NULL; }
   s->elemsize = OcDType_size(dtype); s->dtype = dtype; s->nelem = nelem;
   s->size = s->capacity = nelem * s->elemsize;
   s->data = (char *)malloc(s->size > 0 ? (size_t)s->size : 1);
   s->flags = OC_STORAGE_OWNER; s->refcount = 1; s->finalize = cpu_storage_finalize;
   if (s->data == NULL) { free(s); OcErrorMessage("Insufficient memory to allocate %td bytes", s->size); return NULL; }
   return s;
}
OcStorage *OcIncrefStorage(OcStorage *s) { if (s) s->refcount++; return s; }
void OcDecrefStorage(OcStorage *s)
{  if (s == NULL || --s->refcount > 0) return;
   /* outstanding work on the storage must have finished before its memory goes away (storage.c:51-57) */
   OcStorage_synchronize(s);
   if (s->finalize) s->finalize(s);
   if (s->stream)
   {  OcDevice *d = s->stream->device;
      if (s->event) d->delete_event(d, s->event);
      d->delete_stream(s->stream);
   }
   free(s);
}

/* The reader's stream must see the data that the other stream produced, and the producer's later
   writes must wait for the reader (storage.c:100-160). With one stream per device both are no-ops. */
int OcStorage_startRead(OcStorage *target, OcStorage *read)
{  if (target == read || target->stream == read->stream) return 0;
   if (read->stream == NULL) return 0;                                   /* host memory is always current */
   if (target->stream == NULL) return read->stream->device->sync_stream(read->stream);
   {  OcDevice *d = read->stream->device;
      if (d->record_event(read->event, read->stream) != 0) return -1;
      return target->stream->device->wait_event(target->stream, read->event);
   }
}
int OcStorage_finishRead(OcStorage *target, OcStorage *read)
{  if (target == read || target->stream == read->stream) return 0;
   if (target->stream == NULL || read->stream == NULL) return 0;
   {  OcDevice *d = target->stream->device;
      if (d->record_event(target->event, target->stream) != 0) return -1;
      return read->stream->device->wait_event(read->stream, target->event);
   }
}
int OcStorage_update(OcStorage *storage) { (void)storage; return 0; }
int OcStorage_synchronize(OcStorage *storage)
{  if (storage->stream == NULL) return 0;
   return storage->stream->device->sync_stream(storage->stream);
}

/* ---- tensors ------------------------------------------------------------------- */
static void tensor_update_extent(OcTensor *t)
{  OcSize lo = 0, hi = 0; int i;
   t->nelem = 1;
   for (i = 0; i < t->ndims; i++)
   {  t->nelem *= t->size[i];
      if (t->size[i] > 0)
      {  OcIndex span = (t->size[i] - 1) * t->strides[i];
         if (span < 0) lo += span; else hi += span;
      }
   }
   t->blockOffset = lo;
   t->blockExtent = (t->nelem == 0) ? 0 : (hi - lo + t->elemsize);
}
static OcTensor *tensor_header(int ndims, const OcSize *size, const OcIndex *strides, OcDType dtype)
{  OcTensor *t; int i;
   if (ndims < 0 || ndims > OC_TENSOR_MAX_DIMS) { OcErrorMessage("Invalid number of tensor dimensions (%d)", ndims); return NULL; }
   t = (OcTensor *)calloc(1, sizeof(OcTensor));
   if (t == NULL) { OcErrorMessage("Insufficient memory to allocate the tensor object"); return NULL; }
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
OcTensor *OcTensor_createFromStorage(OcStorage *storage, int ndims, const OcSize *size, const OcIndex *strides, OcSize offset, OcDType dtype)
{  OcTensor *t = tensor_header(ndims, size, strides, dtype);
   if (t == NULL) return NULL;
   if (t->nelem > 0 && (offset + t->blockOffset < 0 || offset + t->blockOffset + t->blockExtent > storage->size))
   {  OcErrorMessage("Tensor extent exceeds the storage size"); free(t->size); free(t->strides); free(t); return NULL; }
   t->storage = OcIncrefStorage(storage); t->offset = offset;
   t->device = storage->stream ? storage->stream->device : OcCPU;
   if (storage->flags & OC_STORAGE_BYTESWAPPED) t->flags |= OC_TENSOR_BYTESWAPPED;
   return t;
}
OcTensor *OcTensor_create(int ndims, const OcSize *size, const OcIndex *strides, OcDType dtype, OcDevice *device)
{  OcTensor *probe = tensor_header(ndims, size, strides, dtype), *t;
   OcStorage *s; OcSize bytes, offset;
   if (probe == NULL) return NULL;
   bytes = probe->blockExtent; offset = -probe->blockOffset;
   free(probe->size); free(probe->strides); free(probe);
   s = OcStorage_create((bytes + OcDType_size(dtype) - 1) / OcDType_size(dtype), dtype, device);
   if (s == NULL) return NULL;
   t = OcTensor_createFromStorage(s, ndims, size, strides, offset, dtype);
   OcDecrefStorage(s);
   return t;
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
   {  OcErrorMessage("Slice out of range"); return NULL; }
   if ((t = OcTensor_shallowCopy(x)) == NULL) return NULL;
   t->offset += start * t->strides[axis];
   t->size[axis] = count; t->strides[axis] *= step;
   tensor_update_extent(t);
   return t;
}
OcTensor *OcTensor_broadcastTo(OcTensor *x, int ndims, const OcSize *size)
{  OcTensor *t; int i;
   if (ndims < x->ndims) { OcErrorMessage("Cannot broadcast to fewer dimensions"); return NULL; }
   for (i = 0; i < x->ndims; i++)
      if (x->size[i] != size[i] && x->size[i] != 1) { OcErrorMessage("Tensor dimensions are not compatible for broadcasting"); return NULL; }
   if ((t = OcTensor_shallowCopy(x)) == NULL) return NULL;
   for (i = 0; i < ndims; i++)
   {  if (i >= x->ndims || (x->size[i] == 1 && size[i] != 1)) t->strides[i] = 0;
      t->size[i] = size[i];
   }
   t->ndims = ndims;
   tensor_update_extent(t);
   return t;
}
void OcTensor_setByteswapped(OcTensor *t, int flag)
{  if (flag) t->flags |= OC_TENSOR_BYTESWAPPED; else t->flags &= ~(OcTensorFlags)OC_TENSOR_BYTESWAPPED; }
int OcTensor_isContiguous(OcTensor *t)
{  OcIndex acc = t->elemsize; int i;
   for (i = 0; i < t->ndims; i++) { if (t->size[i] != 1 && t->strides[i] != acc) return 0; acc *= t->size[i]; }
   return 1;
}

/* ---- caller-side shape analysis ---------------------------------------------- */
int OcShape_sortStrides2(int ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2)
{  int i, j;                      /* insertion sort: ascending strides1, ties by strides2 (shape.c:253-276) */
   for (i = 1; i < ndims; i++)
      for (j = i; j > 0; j--)
      {  int before = (strides1[j - 1] < strides1[j]) || (strides1[j - 1] == strides1[j] && strides2[j - 1] <= strides2[j]);
         OcSize s; OcIndex r;
         if (before) break;
         s = size[j]; size[j] = size[j - 1]; size[j - 1] = s;
         r = strides1[j]; strides1[j] = strides1[j - 1]; strides1[j - 1] = r;
         r = strides2[j]; strides2[j] = strides2[j - 1]; strides2[j - 1] = r;
      }
   return 0;
}
int OcShape_mergeBlocks2(int *ndims, OcSize *size, OcIndex *strides1, OcIndex *strides2)
{  int i, j = 0, n = *ndims;       /* fold dimension i into j when both operands step contiguously (shape.c:334-360) */
   if (n <= 0) return 0;
   for (i = 1; i < n; i++)
   {  if (strides1[i] == strides1[j] * size[j] && strides2[i] == strides2[j] * size[j]) size[j] *= size[i];
      else { j++; size[j] = size[i]; strides1[j] = strides1[i]; strides2[j] = strides2[i]; }
   }
   *ndims = j + 1;
   return 0;
}
/* ocean_solid.c:382-462: kept dimensions (with the destination's strides) and reduced dimensions of an
   axis reduction, unit dimensions dropped, negative strides flipped into the base pointers, sorted and merged.
   The caller adds config->offset1 / offset2 to the source / destination data pointers. */
int OcSolid_analyzeReduceAxis(OcTensor *src, int n, const int *axes, OcTensor *dst, OcSolidReduceAxis *c)
{  int reduced[OC_TENSOR_MAX_DIMS] = { 0 }, i, j = 0, k = 0, keepdims = (src->ndims == dst->ndims);
   OcIndex o1 = 0, o2 = 0, dummy[OC_TENSOR_MAX_DIMS];
   memset(c, 0, sizeof(*c));
   for (i = 0; i < n; i++) reduced[axes[i]] = 1;
   for (i = 0; i < src->ndims; i++)
   {  if (reduced[i]) { if (keepdims) k++; continue; }
      if (src->size[i] != 1)
      {  c->size[j] = src->size[i]; c->strides1[j] = src->strides[i]; c->strides2[j] = dst->strides[k]; j++; }
      k++;
   }
   c->ndims = j;
   for (i = 0, j = 0; i < n; i++)
   {  int a = axes[i];
      if (src->size[a] != 1) { c->rsize[j] = src->size[a]; c->rstrides[j] = src->strides[a]; j++; }
   }
   c->rdims = j;
   for (i = 0; i < c->ndims; i++)                       /* destination strides made non-negative */
      if (c->strides2[i] < 0)
      {  o1 += (c->size[i] - 1) * c->strides1[i]; o2 += (c->size[i] - 1) * c->strides2[i];
         c->strides1[i] = -c->strides1[i]; c->strides2[i] = -c->strides2[i];
      }
   for (i = 0; i < c->rdims; i++)
      if (c->rstrides[i] < 0) { o1 += (c->rsize[i] - 1) * c->rstrides[i]; c->rstrides[i] = -c->rstrides[i]; }
   OcShape_sortStrides2(c->ndims, c->size, c->strides1, c->strides2);
   OcShape_mergeBlocks2(&c->ndims, c->size, c->strides1, c->strides2);
   for (i = 0; i < c->rdims; i++) dummy[i] = c->rstrides[i];
   OcShape_sortStrides2(c->rdims, c->rsize, c->rstrides, dummy);
   for (i = 0; i < c->rdims; i++) dummy[i] = c->rstrides[i];
   OcShape_mergeBlocks2(&c->rdims, c->rsize, c->rstrides, dummy);
   c->offset1 = o1; c->offset2 = o2;
   return 0;
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
