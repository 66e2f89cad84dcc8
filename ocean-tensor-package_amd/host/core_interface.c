/* A small device-independent front end over the module table: what Ocean's interface layer does
 * before it reaches a device function, restricted to the cases the benchmark configurations and
 * the tests exercise. Follows src/core/interface/tensor_itf.c (copy :777-1041, ensure :1226-1304,
 * binary :3983-4133, reductions :5299-5514, axis reductions :5522-5766, gemm :5951-6778) and
 * src/core/generic/tensor_op.c:141-423 (common type, automatic casts, broadcasting, allocation).
 */
#include "core_interface.h"
#include "../../include/ocean_gpu_module.h"
#include <stdlib.h>
#include <string.h>

#define MODULE_OR_FAIL(m, device) OcModuleCore *m = OcModuleCore_forDevice(device); \
   if (m == NULL) OcError(-1, "No core module is registered for device %s", (device) ? (device)->name : "(null)")

/* ---- copy between any two tensors ------------------------------------------------------- */
static int host_copy_same_type(OcTensor *src, OcTensor *dst)
{  OcSize idx[OC_TENSOR_MAX_DIMS] = { 0 }, jdx[OC_TENSOR_MAX_DIMS] = { 0 }, i; int d, es = src->elemsize;
   for (i = 0; i < src->nelem; i++)
   {  OcIndex so = 0, dof = 0;
      for (d = 0; d < src->ndims; d++) so += idx[d] * src->strides[d];
      for (d = 0; d < dst->ndims; d++) dof += jdx[d] * dst->strides[d];
      memcpy(OcTensor_data(dst) + dof, OcTensor_data(src) + so, (size_t)es);
      for (d = 0; d < src->ndims; d++) { if (++idx[d] < src->size[d]) break; idx[d] = 0; }
      for (d = 0; d < dst->ndims; d++) { if (++jdx[d] < dst->size[d]) break; jdx[d] = 0; }
   }
   return 0;
}
int OcTensor_copy(OcTensor *src, OcTensor *dst)
{  if (src->nelem != dst->nelem) OcError(-1, "Mismatch in the number of elements in tensor copy");
   if (src->device == OcCPU && dst->device == OcCPU)
   {  if (src->dtype != dst->dtype || OcTensor_isByteswapped(src) != OcTensor_isByteswapped(dst))
         OcError(-1, "Converting copies between host tensors need the CPU device module, which is not part of this build");
      return host_copy_same_type(src, dst);
   }
   if (src->device == OcCPU) { MODULE_OR_FAIL(m, dst->device); return m->Tensor_copyFromCPU(src, dst); }
   if (dst->device == OcCPU) { MODULE_OR_FAIL(m, src->device); return m->Tensor_copyToCPU(src, dst); }
   {  MODULE_OR_FAIL(m, dst->device); return m->Tensor_copy(src, dst); }
}

/* Replace *tensor by a native-order tensor of the requested type on the requested device when it is not one
   already (tensor_itf.c:1226-1304). The replacement is a new column-major tensor; the old reference is released. */
static int tensor_ensure(OcTensor **tensor, OcDType dtype, OcDevice *device, int temporary)
{  OcTensor *t = *tensor, *r;
   if (dtype == OcDTypeNone) dtype = t->dtype;
   if (device == NULL) device = t->device;
   if (t->dtype == dtype && t->device == device && !OcTensor_isByteswapped(t)) return 0;
   r = temporary ? OcTensor_createTemporary(t->ndims, t->size, NULL, dtype, device) : OcTensor_create(t->ndims, t->size, NULL, dtype, device);
   if (r == NULL) return -1;
   if (OcTensor_copy(t, r) != 0) { OcDecrefTensor(r); return -1; }
   OcDecrefTensor(t);
   *tensor = r;
   return 0;
}
int OcTensor_ensure(OcTensor **tensor, OcDType dtype, OcDevice *device) { return tensor_ensure(tensor, dtype, device, 0); }
int OcTensor_fill(OcTensor *tensor, OcScalar *value)
{  MODULE_OR_FAIL(m, tensor->device);
   return m->Tensor_fill(tensor, value);
}

OcTensor *OcTensor_find(OcTensor *mask)
{  OcModuleCore *m = OcModuleCore_forDevice(mask->device);
   if (m == NULL || m->Tensor_find == NULL) { OcErrorMessage("Find is not supported on device %s", mask->device->name); return NULL; }
   return m->Tensor_find(mask);
}
OcTensor *OcTensor_maskToOffset(OcTensor *mask, OcIndex *strides)
{  OcModuleCore *m = OcModuleCore_forDevice(mask->device);
   if (m == NULL || m->Tensor_maskToOffset == NULL) { OcErrorMessage("Mask-to-offset is not supported on device %s", mask->device->name); return NULL; }
   return m->Tensor_maskToOffset(mask, strides);
}

/* ---- elementwise -------------------------------------------------------------------------- */
typedef int (*oc_binary_fn)(OcTensor *, OcTensor *, OcTensor *);
typedef int (*oc_unary_fn)(OcTensor *, OcTensor *);
#define OC_NBINARY 27
#define OC_NUNARY 40

/* broadcast shape of two tensors: dimensions align from the first; missing trailing dimensions count as 1 */
static int broadcast_shape(OcTensor *a, OcTensor *b, int *ndims, OcSize *size)
{  int i, n = a->ndims > b->ndims ? a->ndims : b->ndims;
   for (i = 0; i < n; i++)
   {  OcSize sa = i < a->ndims ? a->size[i] : 1, sb = i < b->ndims ? b->size[i] : 1;
      if (sa != sb && sa != 1 && sb != 1) OcError(-1, "Tensor dimensions are not compatible (dimension %d: %td and %td)", i, sa, sb);
      size[i] = (sa == 1) ? sb : sa;
   }
   *ndims = n;
   return 0;
}
int OcTensor_binary(int op, OcTensor *src1, OcTensor *src2, OcTensor **dst)
{  OcTensor *a = NULL, *b = NULL, *va = NULL, *vb = NULL, *out = NULL; OcSize size[OC_TENSOR_MAX_DIMS]; int ndims = 0, result = -1;
   OcDevice *device = src1->device != OcCPU ? src1->device : (src2->device != OcCPU ? src2->device : ((*dst) ? (*dst)->device : OcCPU));
   OcDType dtype, dtype2, rtype; oc_binary_fn fn; int is_compare = (op >= 13 && op <= 18), is_shift = (op >= 25), is_logical = (op >= 22 && op <= 24);
   if (op < 0 || op >= OC_NBINARY) OcError(-1, "Invalid binary operation index (%d)", op);
   {  MODULE_OR_FAIL(m, device);
      fn = ((oc_binary_fn *)&m->Tensor_add)[op];
      if (fn == NULL) OcError(-1, "Tensor operation is not supported on device %s", device->name);
   }
   /* common type of the operands; shifts keep the type of the first operand and take int8 counts,
      integer powers take int16 exponents, logical operations work on bool */
   dtype = is_shift ? src1->dtype : OcDType_getCommonType(src1->dtype, src2->dtype);
   if (is_logical) dtype = OcDTypeBool;
   dtype2 = dtype;
   if (is_shift) dtype2 = OcDTypeInt8;
   if (op == 6)
   {  /* power (tensor_itf.c:4736-4760): the base keeps its type (widened by a given destination's); two integer
         operands take an int16 exponent, anything else the common type for both */
      dtype = (*dst) ? OcDType_getCommonType(src1->dtype, (*dst)->dtype) : src1->dtype;
      if (!OcDType_isFloat(dtype) && !OcDType_isFloat(src2->dtype)) dtype2 = OcDTypeInt16;
      else { dtype = OcDType_getCommonType(dtype, src2->dtype); dtype2 = dtype; }
   }
   rtype = is_compare ? OcDTypeBool : dtype;
   a = OcIncrefTensor(src1); b = OcIncrefTensor(src2);
   /* converted operands live in the device's ring of temporary storages: releasing them does not wait for the device */
   if (tensor_ensure(&a, dtype, device, 1) != 0 || tensor_ensure(&b, dtype2, device, 1) != 0) goto final;
   if (broadcast_shape(a, b, &ndims, size) != 0) goto final;
   if ((va = OcTensor_broadcastTo(a, ndims, size)) == NULL || (vb = OcTensor_broadcastTo(b, ndims, size)) == NULL) goto final;
   if (*dst == NULL)
   {  if ((out = OcTensor_create(ndims, size, NULL, rtype, device)) == NULL) goto final;
      result = fn(va, vb, out);
      if (result == 0) { *dst = out; out = NULL; }
   }
   else if ((*dst)->dtype == rtype && (*dst)->device == device && !OcTensor_isByteswapped(*dst))
   {  OcTensor *vd = OcTensor_broadcastTo(*dst, ndims, size);          /* shape check: must not actually broadcast */
      int i, ok = (vd != NULL);
      for (i = 0; ok && i < ndims; i++) if ((i < (*dst)->ndims ? (*dst)->size[i] : 1) != size[i]) ok = 0;
      if (!ok) { if (vd) OcDecrefTensor(vd); if (vd) OcErrorMessage("Destination size does not match the operands"); goto final; }
      result = fn(va, vb, vd);
      OcDecrefTensor(vd);
   }
   else
   {  /* compute in the working type, then convert into the caller's destination */
      if ((out = OcTensor_create(ndims, size, NULL, rtype, device)) == NULL) goto final;
      if (fn(va, vb, out) != 0) goto final;
      result = OcTensor_copy(out, *dst);
   }
final:
   if (out) OcDecrefTensor(out);
   if (va) OcDecrefTensor(va);
   if (vb) OcDecrefTensor(vb);
   if (a) OcDecrefTensor(a);
   if (b) OcDecrefTensor(b);
   return result;
}
int OcTensor_unary(int op, OcTensor *src, OcTensor **dst)
{  OcTensor *a = NULL, *out = NULL; oc_unary_fn fn; int result = -1; OcDType rtype;
   if (op < 0 || op >= OC_NUNARY) OcError(-1, "Invalid unary operation index (%d)", op);
   {  MODULE_OR_FAIL(m, src->device);
      fn = ((oc_unary_fn *)&m->Tensor_negative)[op];
      if (fn == NULL) OcError(-1, "Tensor operation is not supported on device %s", src->device->name);
   }
   a = OcIncrefTensor(src);
   {  /* the negative of an unsigned tensor is taken in its signed type (tensor_itf.c:3637-3651, signed types of src/base/dtype.c:57-61) */
      static const OcDType signed_of[5] = { OcDTypeInt16, OcDTypeInt16, OcDTypeInt32, OcDTypeInt64, OcDTypeDouble };
      OcDType work = a->dtype;
      if (op == 0 && work >= OcDTypeUInt8 && work <= OcDTypeUInt64) work = signed_of[work];
      if (op == 2) work = OcDTypeBool;                                      /* logical not works on truth values (tensor_itf.c:3669-3676) */
      if (OcTensor_ensure(&a, work, a->device) != 0) goto final;
   }
   rtype = a->dtype;
   if (op >= 35) rtype = OcDTypeBool;                                       /* isinf ... isneginf */
   if (op == 28 && OcDType_isComplex(a->dtype)) rtype = OcDType_getBaseType(a->dtype);   /* absolute of complex is real */
   if (*dst && (*dst)->dtype == rtype && (*dst)->device == a->device && !OcTensor_isByteswapped(*dst)) result = fn(a, *dst);
   else
   {  if ((out = OcTensor_create(a->ndims, a->size, NULL, rtype, a->device)) == NULL) goto final;
      if ((result = fn(a, out)) != 0) goto final;
      if (*dst) result = OcTensor_copy(out, *dst); else { *dst = out; out = NULL; }
   }
final:
   if (out) OcDecrefTensor(out);
   if (a) OcDecrefTensor(a);
   return result;
}

/* ---- reductions ------------------------------------------------------------------------------ */
int OcTensor_reduceAll(int which, OcTensor *tensor, double p, OcScalar *result)
{  OcTensor *a = OcIncrefTensor(tensor); int r = -1;
   if (OcTensor_ensure(&a, a->dtype, a->device) == 0)          /* native byte order (tensor_itf.c:5308) */
   {  OcModuleCore *m = OcModuleCore_forDevice(a->device);
      if (m == NULL) OcErrorMessage("No core module is registered for device %s", a->device->name);
      else switch (which)
      {  case 15: r = m->Tensor_sum(a, result); break;        case 16: r = m->Tensor_sumNaN(a, result); break;
         case 17: r = m->Tensor_prod(a, result); break;       case 18: r = m->Tensor_prodNaN(a, result); break;
         case 19: r = m->Tensor_sumAbs(a, result); break;     case 20: r = m->Tensor_sumAbsNaN(a, result); break;
         case 21: r = m->Tensor_maximum(a, result); break;    case 22: r = m->Tensor_minimum(a, result); break;
         case 23: r = m->Tensor_maximumAbs(a, result); break; case 24: r = m->Tensor_minimumAbs(a, result); break;
         case 25: r = m->Tensor_norm(a, p, result); break;    case 26: r = m->Tensor_normNaN(a, p, result); break;
         case 27: r = m->Tensor_norm2(a, result); break;      case 28: r = m->Tensor_norm2NaN(a, result); break;
         default: OcErrorMessage("Reduction %d does not return a scalar", which);
      }
   }
   OcDecrefTensor(a);
   return r;
}
/* the logical reductions (any, all, allFinite, anyInf, anyNaN: which = 0 ... 4) and the counts (nnz, nnzNaN: 5, 6) of
   tensor_itf.c:5299-5400, through the same table */
int OcTensor_reduceLogical(int which, OcTensor *tensor, int *result)
{  OcTensor *a = OcIncrefTensor(tensor); int r = -1;
   if (OcTensor_ensure(&a, a->dtype, a->device) == 0)
   {  OcModuleCore *m = OcModuleCore_forDevice(a->device);
      if (m == NULL) OcErrorMessage("No core module is registered for device %s", a->device->name);
      else switch (which)
      {  case 0: r = m->Tensor_any(a, result); break;        case 1: r = m->Tensor_all(a, result); break;
         case 2: r = m->Tensor_allFinite(a, result); break;  case 3: r = m->Tensor_anyInf(a, result); break;
         case 4: r = m->Tensor_anyNaN(a, result); break;
         default: OcErrorMessage("Reduction %d does not return a truth value", which);
      }
   }
   OcDecrefTensor(a);
   return r;
}
int OcTensor_reduceCount(int which, OcTensor *tensor, OcUInt64 *result)
{  OcTensor *a = OcIncrefTensor(tensor); int r = -1;
   if (OcTensor_ensure(&a, a->dtype, a->device) == 0)
   {  OcModuleCore *m = OcModuleCore_forDevice(a->device);
      if (m == NULL) OcErrorMessage("No core module is registered for device %s", a->device->name);
      else if (which == 5) r = m->Tensor_nnz(a, result);
      else if (which == 6) r = m->Tensor_nnzNaN(a, result);
      else OcErrorMessage("Reduction %d does not return a count", which);
   }
   OcDecrefTensor(a);
   return r;
}
int OcTensor_sum(OcTensor *t, OcScalar *r)     { return OcTensor_reduceAll(15, t, 0.0, r); }
int OcTensor_maximum(OcTensor *t, OcScalar *r) { return OcTensor_reduceAll(21, t, 0.0, r); }
int OcTensor_norm2(OcTensor *t, OcScalar *r)   { return OcTensor_reduceAll(27, t, 0.0, r); }

typedef int (*oc_axis_fn)(OcTensor *, int, int *, OcTensor *);
static OcDType reduce_result_type(int which, OcDType d)
{  int isbool = (d == OcDTypeBool), isuint = (d >= OcDTypeUInt8 && d <= OcDTypeUInt64), issint = (d >= OcDTypeInt8 && d <= OcDTypeInt64);
   OcDType mag = OcDType_isComplex(d) ? OcDType_getBaseType(d) : (issint ? (OcDType)(d - 4) : d);
   if (which <= 4) return OcDTypeBool;
   if (which <= 6) return OcDTypeUInt64;
   if (which >= 15 && which <= 18) return (isbool || isuint) ? OcDTypeUInt64 : (issint ? OcDTypeInt64 : d);
   if (which == 19 || which == 20) return (isbool || isuint || issint) ? OcDTypeUInt64 : mag;
   if (which == 21 || which == 22) return d;
   if (which == 23 || which == 24) return mag;
   return (isbool || isuint || issint) ? OcDTypeDouble : mag;
}
/* axes validated, made unique and non-negative (tensor_itf.c:5537-5554); dst created when *dst is NULL */
int OcTensor_axisReduce(int which, OcTensor *src, int n, int *axes, int keepdims, double p, OcTensor **dst)
{  int flag[OC_TENSOR_MAX_DIMS] = { 0 }, ax[OC_TENSOR_MAX_DIMS], i, j, nd = 0, r = -1; OcSize size[OC_TENSOR_MAX_DIMS];
   OcTensor *a, *out = NULL; OcModuleCore *m; OcDType rtype;
   static const int order[] = { 0, 1, 2, 3, 4, 5, 6, 15, 17, 16, 18, 19, 20, 22, 21, 24, 23, 27, 28 };   /* table order of the axis block */
   for (i = 0, j = 0; i < n; i++)
   {  int k = axes[i] < 0 ? axes[i] + src->ndims : axes[i];
      if (k < 0 || k >= src->ndims) OcError(-1, "Axis index %d out of range", axes[i]);
      if (flag[k]) OcError(-1, "Repeated axis index %d", axes[i]);
      flag[k] = 1; ax[j++] = k;
   }
   for (i = 0; i < src->ndims; i++) { if (!flag[i]) size[nd++] = src->size[i]; else if (keepdims) size[nd++] = 1; }
   a = OcIncrefTensor(src);
   if (OcTensor_ensure(&a, a->dtype, a->device) != 0) goto final;
   if ((m = OcModuleCore_forDevice(a->device)) == NULL) { OcErrorMessage("No core module is registered for device %s", a->device->name); goto final; }
   rtype = reduce_result_type(which, a->dtype);
   if (*dst && (*dst)->dtype == rtype && (*dst)->device == a->device && !OcTensor_isByteswapped(*dst)) out = OcIncrefTensor(*dst);
   else if ((out = OcTensor_create(nd, size, NULL, rtype, a->device)) == NULL) goto final;
   if (out->ndims != nd) { OcErrorMessage("Destination has %d dimensions, expected %d", out->ndims, nd); goto final; }
   for (i = 0; i < nd; i++) if (out->size[i] != size[i]) { OcErrorMessage("Destination size mismatch in dimension %d", i); goto final; }
   if (which == 25) r = m->Tensor_axisNorm(a, p, j, ax, out);
   else if (which == 26) r = m->Tensor_axisNormNaN(a, p, j, ax, out);
   else
   {  oc_axis_fn fn = NULL;
      for (i = 0; i < (int)(sizeof(order) / sizeof(order[0])); i++) if (order[i] == which) fn = ((oc_axis_fn *)&m->Tensor_axisAny)[i];
      if (fn == NULL) { OcErrorMessage("Axis reduction %d is not available", which); goto final; }
      r = fn(a, j, ax, out);
   }
   if (r == 0 && *dst == NULL) { *dst = out; out = NULL; }
   else if (r == 0 && *dst != out) r = OcTensor_copy(out, *dst);
final:
   if (out) OcDecrefTensor(out);
   OcDecrefTensor(a);
   return r;
}

/* ---- GEMM ---------------------------------------------------------------------------------------- */
/* float -> half as Ocean converts it (solid/src/base/generic/half.c): values below 2^-15 become zero, ties round away from
   zero, NaN becomes 0x7F00 */
static OcUInt16 half_bits(float f)
{  unsigned int raw, d, s, ex; memcpy(&raw, &f, 4);
   d = raw & 0x007FFFFFu; s = (raw >> 16) & 0x8000u; ex = (raw >> 23) & 0xFFu;
   if (ex < 112u) return 0;
   if (ex > 143u) return (OcUInt16)((ex == 255u && d != 0) ? 0x7F00u : (s | 0x7C00u));
   {  unsigned int v = (((ex - 112u) << 10) | (d >> 13) | s) & 0xFFFFu;
      if ((d & 0x1FFFu) >= 0x1000u) v++;
      return (OcUInt16)v;
   }
}
/* C <- alpha op(A) op(B) + beta C. Operands are brought to one type; an operand whose columns are not
   contiguous is either used through the opposite transposition (when its rows are contiguous) or copied
   (tensor_itf.c:6137-6778); alpha and beta become one-element host tensors of that type (:5951-5992). */
static OcTensor *scalar_tensor(OcScalar *s, OcDType dtype, double fallback)
{  OcSize one = 1; OcTensor *t = OcTensor_create(0, &one, NULL, dtype, OcCPU); char *p;
   double re = fallback, im = 0;
   if (t == NULL) return NULL;
   if (s)
      switch (s->dtype)
      {  case OcDTypeBool: re = s->value.sBool; break;      case OcDTypeUInt8: re = s->value.sUInt8; break;
         case OcDTypeUInt16: re = s->value.sUInt16; break;  case OcDTypeUInt32: re = s->value.sUInt32; break;
         case OcDTypeUInt64: re = (double)s->value.sUInt64; break; case OcDTypeInt8: re = s->value.sInt8; break;
         case OcDTypeInt16: re = s->value.sInt16; break;    case OcDTypeInt32: re = s->value.sInt32; break;
         case OcDTypeInt64: re = (double)s->value.sInt64; break;   case OcDTypeFloat: re = s->value.sFloat; break;
         case OcDTypeDouble: re = s->value.sDouble; break;
         case OcDTypeCFloat: re = s->value.sCFloat.real; im = s->value.sCFloat.imag; break;
         case OcDTypeCDouble: re = s->value.sCDouble.real; im = s->value.sCDouble.imag; break;
         default: OcErrorMessage("Half-precision scalars are not supported by this front end"); OcDecrefTensor(t); return NULL;
      }
   p = OcTensor_data(t);
   switch (dtype)
   {  case OcDTypeBool: *(OcBool *)p = (re != 0); break;       case OcDTypeUInt8: *(OcUInt8 *)p = (OcUInt8)re; break;
      case OcDTypeUInt16: *(OcUInt16 *)p = (OcUInt16)re; break; case OcDTypeUInt32: *(OcUInt32 *)p = (OcUInt32)re; break;
      case OcDTypeUInt64: *(OcUInt64 *)p = (OcUInt64)re; break; case OcDTypeInt8: *(OcInt8 *)p = (OcInt8)re; break;
      case OcDTypeInt16: *(OcInt16 *)p = (OcInt16)re; break;   case OcDTypeInt32: *(OcInt32 *)p = (OcInt32)re; break;
      case OcDTypeInt64: *(OcInt64 *)p = (OcInt64)re; break;   case OcDTypeFloat: *(OcFloat *)p = (OcFloat)re; break;
      case OcDTypeDouble: *(OcDouble *)p = re; break;
      case OcDTypeCFloat: ((OcCFloat *)p)->real = (OcFloat)re; ((OcCFloat *)p)->imag = (OcFloat)im; break;
      case OcDTypeCDouble: ((OcCDouble *)p)->real = re; ((OcCDouble *)p)->imag = im; break;
      case OcDTypeHalf: *(OcUInt16 *)p = half_bits((float)re); break;
      default: OcErrorMessage("GEMM scalars of type %s are not supported by this front end", OcDType_name(dtype)); OcDecrefTensor(t); return NULL;
   }
   return t;
}
/* value converted to the given type (OcScalar_castTo, src/base/scalar.c), through the one-element tensor above */
static int scalar_cast(OcScalar *value, OcDType dtype, OcScalar *result)
{  OcTensor *t;
   if (value->dtype == dtype) { *result = *value; return 0; }
   if ((t = scalar_tensor(value, dtype, 0)) == NULL) return -1;
   memset(result, 0, sizeof(*result));
   result->dtype = dtype;
   memcpy(&result->value, OcTensor_data(t), (size_t)t->elemsize);
   OcDecrefTensor(t);
   return 0;
}
/* tensor_itf.c:2788-2826: NaN entries are replaced by the value in the tensor's type; integer tensors are left alone */
int OcTensor_fillNaN(OcTensor *tensor, OcScalar *value)
{  OcScalar v; MODULE_OR_FAIL(m, tensor->device);
   if (m->Tensor_fillNaN == NULL) OcError(-1, "Tensor fill NaN is not supported on device %s", tensor->device->name);
   if (!OcDType_isFloat(tensor->dtype)) return 0;
   if (scalar_cast(value, tensor->dtype, &v) != 0) return -1;
   return m->Tensor_fillNaN(tensor, &v);
}
/* tensor_itf.c:2864-2908: the value is converted to the tensor's type, the mask is broadcast to the tensor's shape
   and brought to bool on the tensor's device, then the device function runs */
int OcTensor_maskedFill(OcTensor *tensor, OcTensor *mask, OcScalar *value)
{  OcScalar v; OcTensor *view = NULL, *m1 = NULL; int result = -1;
   MODULE_OR_FAIL(m, tensor->device);
   if (m->Tensor_maskedFill == NULL) OcError(-1, "Tensor masked fill is not supported on device %s", tensor->device->name);
   if (scalar_cast(value, tensor->dtype, &v) != 0) return -1;
   m1 = OcIncrefTensor(mask);
   if (tensor_ensure(&m1, OcDTypeBool, tensor->device, 1) != 0) goto final;
   if ((view = OcTensor_broadcastTo(m1, tensor->ndims, tensor->size)) == NULL) goto final;
   if (OcTensor_isByteswapped(tensor))
   {  /* the stored bytes are in the other order: fill with the swapped value (each part of a complex value by itself) */
      int parts = OcDType_isComplex(tensor->dtype) ? 2 : 1, w = tensor->elemsize / parts, i, j; char *b = (char *)&v.value;
      for (j = 0; j < parts; j++) for (i = 0; i < w / 2; i++) { char c = b[j * w + i]; b[j * w + i] = b[j * w + w - 1 - i]; b[j * w + w - 1 - i] = c; }
   }
   result = m->Tensor_maskedFill(tensor, view, &v);
final:
   if (view) OcDecrefTensor(view);
   if (m1) OcDecrefTensor(m1);
   return result;
}
/* value(i) = offset + i * step over the flat index, first dimension fastest (the building block of OcTensor_range and
   OcTensor_linspace, tensor_itf.c:2965-3075) */
int OcTensor_stepsInt64(OcTensor *tensor, OcInt64 offset, OcInt64 step)
{  MODULE_OR_FAIL(m, tensor->device);
   if (m->Tensor_stepsInt64 == NULL) OcError(-1, "Tensor steps is not supported on device %s", tensor->device->name);
   return m->Tensor_stepsInt64(tensor, offset, step);
}
int OcTensor_stepsDouble(OcTensor *tensor, OcDouble offset, OcDouble step)
{  MODULE_OR_FAIL(m, tensor->device);
   if (m->Tensor_stepsDouble == NULL) OcError(-1, "Tensor steps is not supported on device %s", tensor->device->name);
   return m->Tensor_stepsDouble(tensor, offset, step);
}
/* leading dimension of a matrix operand, flipping the mode when only its rows are contiguous */
static int gemm_operand(OcTensor **t, char *mode, OcIndex *ld, int complex_type)
{  OcTensor *x = *t; int es = x->elemsize;
   if (x->ndims < 2) OcError(-1, "Matrix multiplication needs tensors of at least two dimensions");
   if ((x->size[0] == 1 || x->strides[0] == es) && (x->size[1] == 1 || (x->strides[1] >= x->size[0] * es && x->strides[1] % es == 0)))
   {  *ld = (x->size[1] == 1) ? (x->size[0] > 0 ? x->size[0] : 1) : x->strides[1] / es; return 0; }
   if ((x->size[1] == 1 || x->strides[1] == es) && (x->size[0] == 1 || (x->strides[0] >= x->size[1] * es && x->strides[0] % es == 0)) && !(complex_type && *mode == 'C'))
   {  /* rows contiguous: the stored matrix is the transpose */
      OcTensor *v = OcTensor_transpose(x);
      if (v == NULL) return -1;
      *ld = (v->size[1] == 1) ? (v->size[0] > 0 ? v->size[0] : 1) : v->strides[1] / es;
      *mode = (*mode == 'N') ? 'T' : 'N';
      OcDecrefTensor(x); *t = v;
      return 0;
   }
   {  OcTensor *r = OcTensor_create(x->ndims, x->size, NULL, x->dtype, x->device);
      if (r == NULL) return -1;
      if (OcTensor_copy(x, r) != 0) { OcDecrefTensor(r); return -1; }
      OcDecrefTensor(x); *t = r; *ld = r->size[0] > 0 ? r->size[0] : 1;
      return 0;
   }
}
/* C <- alpha * op(A) * op(B) + beta * C on the first two dimensions; the dimensions beyond them index independent
   products and broadcast between A and B (size 1 or absent: shared), as in Ocean's interface (tensor_itf.c:6433-6750) */
/* alphaT / betaT: NULL (then the OcScalar, or 1 and 0), or tensors of one element per product: dimensions 0 and 1 of
   size 1, the dimensions beyond them broadcast with those of A and B (tensor_itf.c:6433-6470) */
static int gemm_core(OcScalar *alpha, OcTensor *alphaT, OcTensor *A, char modeA, OcTensor *B, char modeB, OcScalar *beta, OcTensor *betaT, OcTensor **C)
{  OcTensor *a = OcIncrefTensor(A), *b = OcIncrefTensor(B), *c = NULL, *ta = NULL, *tb = NULL, *v; int result = -1, i, nd;
   OcDevice *device = A->device != OcCPU ? A->device : B->device; OcDType dtype = OcDType_getCommonType(A->dtype, B->dtype), halftype = OcDTypeNone;
   OcSize M, N, K, K2, csize[OC_TENSOR_MAX_DIMS], asize[OC_TENSOR_MAX_DIMS], bsize[OC_TENSOR_MAX_DIMS]; OcIndex ldA, ldB, ldC; OcModuleCore *m = OcModuleCore_forDevice(device);
   if (*C) dtype = OcDType_getCommonType(dtype, (*C)->dtype);
   if (m == NULL) { OcErrorMessage("No core module is registered for device %s", device->name); goto final; }
   /* half types the device cannot multiply are computed in float and converted back (tensor_itf.c:6388-6400, 6756-6758) */
   if ((dtype == OcDTypeHalf || dtype == OcDTypeCHalf) && !m->Tensor_gemmSupportedOn(device, dtype))
   {  halftype = dtype; dtype = (dtype == OcDTypeHalf) ? OcDTypeFloat : OcDTypeCFloat; }
   if (!m->Tensor_gemmSupportedOn(device, dtype)) { OcErrorMessage("Matrix multiplication is not supported for type %s on %s", OcDType_name(dtype), device->name); goto final; }
   if (A->ndims < 2 || B->ndims < 2) { OcErrorMessage("Matrix multiplication needs tensors of at least two dimensions"); goto final; }
   M = (modeA == 'N') ? A->size[0] : A->size[1]; K = (modeA == 'N') ? A->size[1] : A->size[0];
   K2 = (modeB == 'N') ? B->size[0] : B->size[1]; N = (modeB == 'N') ? B->size[1] : B->size[0];
   if (K != K2) { OcErrorMessage("Inner dimensions do not match (%td and %td)", K, K2); goto final; }
   nd = A->ndims > B->ndims ? A->ndims : B->ndims;
   if (alphaT && alphaT->ndims > nd) nd = alphaT->ndims;
   if (betaT && betaT->ndims > nd) nd = betaT->ndims;
   csize[0] = M; csize[1] = N;
   for (i = 2; i < nd; i++)
   {  OcTensor *ops[4] = { A, B, alphaT, betaT }; int k;
      csize[i] = 1;
      for (k = 0; k < 4; k++)
      {  OcSize sk = (ops[k] && i < ops[k]->ndims) ? ops[k]->size[i] : 1;
         if (sk != 1 && csize[i] != 1 && sk != csize[i]) { OcErrorMessage("Dimension %d of the operands is not compatible (%td and %td)", i, csize[i], sk); goto final; }
         if (sk != 1) csize[i] = sk;
      }
   }
   for (i = 0; i < 2; i++)
      if ((alphaT && i < alphaT->ndims && alphaT->size[i] != 1) || (betaT && i < betaT->ndims && betaT->size[i] != 1))
      {  OcErrorMessage("The scalars of a matrix product must have size one in the first two dimensions"); goto final; }
   if (OcTensor_ensure(&a, dtype, device) != 0 || OcTensor_ensure(&b, dtype, device) != 0) goto final;
   if (gemm_operand(&a, &modeA, &ldA, OcDType_isComplex(dtype)) != 0 || gemm_operand(&b, &modeB, &ldB, OcDType_isComplex(dtype)) != 0) goto final;
   /* all operands get the same number of dimensions; shared ones have stride zero */
   asize[0] = a->size[0]; asize[1] = a->size[1]; bsize[0] = b->size[0]; bsize[1] = b->size[1];
   for (i = 2; i < nd; i++) asize[i] = bsize[i] = csize[i];
   if ((v = OcTensor_broadcastTo(a, nd, asize)) == NULL) goto final;
   OcDecrefTensor(a); a = v;
   if ((v = OcTensor_broadcastTo(b, nd, bsize)) == NULL) goto final;
   OcDecrefTensor(b); b = v;
   if (*C == NULL) { if ((c = OcTensor_create(nd, csize, NULL, dtype, device)) == NULL) goto final; }
   else
   {  int same = ((*C)->ndims == nd);
      c = OcIncrefTensor(*C);
      for (i = 0; same && i < nd; i++) if (c->size[i] != csize[i]) same = 0;
      if (!same) { OcErrorMessage("Destination size does not match the product"); goto final; }
      for (i = 2; same && i < nd; i++) if (c->size[i] > 1 && c->strides[i] == 0) same = 0;      /* products must not share their destination */
      if (c->dtype != dtype || c->device != device || OcTensor_isByteswapped(c) || (M > 1 && c->strides[0] != c->elemsize) ||
          (N > 1 && (c->strides[1] < M * c->elemsize || c->strides[1] % c->elemsize != 0)) || !same)
      {  if (OcTensor_ensure(&c, dtype, device) != 0) goto final;
         if (c == *C)                                   /* same type but unusable layout: work on a dense copy */
         {  OcTensor *r = OcTensor_create(nd, csize, NULL, dtype, device);
            if (r == NULL || OcTensor_copy(c, r) != 0) { if (r) OcDecrefTensor(r); goto final; }
            OcDecrefTensor(c); c = r;
         }
      }
   }
   ldC = (N > 1) ? c->strides[1] / c->elemsize : (M > 0 ? M : 1);
   /* scalars: both on the host or both on the device (the module reads the flag from alpha, tensor_blas_gpu.c:108-120) */
   {  OcDevice *sdev = (alphaT && alphaT->device != OcCPU) || (betaT && betaT->device != OcCPU) ? device : OcCPU;
      OcSize ssize[OC_TENSOR_MAX_DIMS]; int k;
      ssize[0] = ssize[1] = 1; for (k = 2; k < nd; k++) ssize[k] = csize[k];
      ta = alphaT ? OcIncrefTensor(alphaT) : scalar_tensor(alpha, dtype, 1.0);
      tb = betaT ? OcIncrefTensor(betaT) : scalar_tensor(beta, dtype, 0.0);
      if (ta == NULL || tb == NULL) goto final;
      if (OcTensor_ensure(&ta, dtype, sdev) != 0 || OcTensor_ensure(&tb, dtype, sdev) != 0) goto final;
      if ((v = OcTensor_broadcastTo(ta, nd, ssize)) == NULL) goto final;
      OcDecrefTensor(ta); ta = v;
      if ((v = OcTensor_broadcastTo(tb, nd, ssize)) == NULL) goto final;
      OcDecrefTensor(tb); tb = v;
      if (sdev != OcCPU && (OcTensor_startRead(c, ta) != 0 || OcTensor_startRead(c, tb) != 0)) goto final;
   }
   /* the caller runs the stream protocol around Tensor_gemm (tensor_itf.c:6727-6750) */
   if (OcTensor_startRead(c, a) != 0 || OcTensor_startRead(c, b) != 0) goto final;
   result = m->Tensor_gemm(M, N, K, modeA, modeB, ta, a, ldA, b, ldB, tb, c, ldC);
   if (result == 0 && (OcTensor_update(c) != 0 || OcTensor_finishRead(c, a) != 0 || OcTensor_finishRead(c, b) != 0)) result = -1;
   if (result == 0 && ta->device != OcCPU && (OcTensor_finishRead(c, ta) != 0 || OcTensor_finishRead(c, tb) != 0)) result = -1;
   if (result == 0 && *C == NULL && halftype != OcDTypeNone) result = OcTensor_ensure(&c, halftype, device);
   if (result == 0 && *C == NULL) { *C = c; c = NULL; }
   else if (result == 0 && c != *C) result = OcTensor_copy(c, *C);
final:
   if (ta) OcDecrefTensor(ta);
   if (tb) OcDecrefTensor(tb);
   if (c) OcDecrefTensor(c);
   OcDecrefTensor(a); OcDecrefTensor(b);
   return result;
}
int OcTensor_mtimes(OcTensor *A, OcTensor *B, OcTensor **C) { return OcTensor_gemm(NULL, A, 'N', B, 'N', NULL, C); }

int OcTensor_gemm(OcScalar *alpha, OcTensor *A, char modeA, OcTensor *B, char modeB, OcScalar *beta, OcTensor **C)
{  return gemm_core(alpha, NULL, A, modeA, B, modeB, beta, NULL, C); }
int OcTensor_gemmTensors(OcTensor *alpha, OcTensor *A, char modeA, OcTensor *B, char modeB, OcTensor *beta, OcTensor **C)
{  return gemm_core(NULL, alpha, A, modeA, B, modeB, NULL, beta, C); }
/* ---- index operations through the table (src/core/interface/index_itf.c, tensor_itf.c:2359-2700) ----------------- */
/* indices: int64 tensor [k, n] on the tensor's device: n index tuples for the first k dimensions of `tensor` (negative
   values count from the end). Builds the view the interface builds -- one offset table per indexed dimension, made by
   Tensor_addIfNegative + Tensor_indexToOffset on storages (and streams) of their own -- and hands it to the module. */
static int index_view(OcTensor *tensor, OcTensor *indices, OcTensorIndexView *view, OcTensor **work, OcSize *vsize, OcIndex *vstrides, int *vnd)
{  OcModuleCore *m = OcModuleCore_forDevice(tensor->device); int k, d; OcSize n;
   if (m == NULL) OcError(-1, "No core module is registered for device %s", tensor->device->name);
   if (indices->dtype != OcDTypeInt64 || indices->ndims != 2 || indices->device != tensor->device) OcError(-1, "Indices must be an int64 tensor [k, n] on the tensor's device");
   k = (int)indices->size[0]; n = indices->size[1];
   if (k < 1 || k > tensor->ndims) OcError(-1, "Number of index dimensions out of range");
   memset(view, 0, sizeof(*view));
   /* view dimensions: one of size n for the tuples, then the dimensions of the tensor that are not indexed; every
      indexed dimension but the first becomes a dimension of size 1 whose table is broadcast -- here the k tables are
      folded into ONE table of byte offsets (indexToOffset multiplies by the strides and sums over the k rows) */
   *vnd = 1 + tensor->ndims - k;
   vsize[0] = n; vstrides[0] = 0;
   for (d = k; d < tensor->ndims; d++) { vsize[1 + d - k] = tensor->size[d]; vstrides[1 + d - k] = tensor->strides[d]; }
   {  OcTensor *idx = OcTensor_create(2, indices->size, NULL, OcDTypeInt64, tensor->device), *off; OcInt64 strides[OC_TENSOR_MAX_DIMS]; OcScalar s;
      OcSize one = n;
      if (idx == NULL) return -1;
      if (OcTensor_copy(indices, idx) != 0) { OcDecrefTensor(idx); return -1; }
      for (d = 0; d < k; d++)              /* negative indices: add the dimension's size, row by row */
      {  OcTensor *row = OcTensor_slice(idx, 0, d, 1, 1);
         /* every index must lie in [-size, size): checked with the module's own full reductions before anything is
            addressed through it, as the interface does when an index is bound (index_itf.c:1311-1336, which keeps the
            minimum and maximum of every index row) */
         if (row != NULL && n > 0)
         {  OcScalar lo, hi;
            if (m->Tensor_minimum == NULL || m->Tensor_maximum == NULL || m->Tensor_minimum(row, &lo) != 0 || m->Tensor_maximum(row, &hi) != 0)
            {  OcDecrefTensor(row); OcDecrefTensor(idx); OcError(-1, "Could not determine the range of the tensor indices"); }
            if (lo.value.sInt64 < -(OcInt64)tensor->size[d] || hi.value.sInt64 >= (OcInt64)tensor->size[d])
            {  long bad = (long)((lo.value.sInt64 < -(OcInt64)tensor->size[d]) ? lo.value.sInt64 : hi.value.sInt64);
               OcDecrefTensor(row); OcDecrefTensor(idx);
               OcError(-1, "Tensor index (%ld) out of range (%lu) at dimension %d", bad, (unsigned long)tensor->size[d], d);
            }
         }
         s.dtype = OcDTypeInt64; s.value.sInt64 = tensor->size[d];
         if (row == NULL || m->Tensor_addIfNegative(row, &s) != 0) { if (row) OcDecrefTensor(row); OcDecrefTensor(idx); return -1; }
         OcDecrefTensor(row);
         strides[d] = tensor->strides[d];
      }
      if ((off = OcTensor_create(1, &one, NULL, OcDTypeInt64, tensor->device)) == NULL) { OcDecrefTensor(idx); return -1; }
      if (m->Tensor_indexToOffset(idx, strides, off) != 0) { OcDecrefTensor(idx); OcDecrefTensor(off); return -1; }
      OcDecrefTensor(idx);
      *work = off;
   }
   return 0;
}
int OcTensor_getIndexed(OcTensor *tensor, OcTensor *indices, OcTensor **dst)
{  OcTensorIndexView view; OcTensor *off = NULL, *v = NULL, *out = NULL, *offsets[OC_TENSOR_MAX_DIMS] = { 0 }; OcSize vsize[OC_TENSOR_MAX_DIMS]; OcIndex vstrides[OC_TENSOR_MAX_DIMS];
   int vnd, result = -1; OcModuleCore *m = OcModuleCore_forDevice(tensor->device);
   if (index_view(tensor, indices, &view, &off, vsize, vstrides, &vnd) != 0) return -1;
   if ((v = OcTensor_createFromStorage(tensor->storage, vnd, vsize, vstrides, tensor->offset, tensor->dtype)) == NULL) goto final;
   offsets[0] = off; view.ndims = vnd; view.view = v; view.offsets = offsets;
   if ((out = OcTensor_create(vnd, vsize, NULL, tensor->dtype, tensor->device)) == NULL) goto final;
   if ((result = m->Tensor_getIndex(&view, out)) == 0) { *dst = out; out = NULL; }
final:
   if (out) OcDecrefTensor(out);
   if (v) OcDecrefTensor(v);
   if (off) OcDecrefTensor(off);
   return result;
}
int OcTensor_setIndexed(OcTensor *tensor, OcTensor *indices, OcTensor *src)
{  OcTensorIndexView view; OcTensor *off = NULL, *v = NULL, *offsets[OC_TENSOR_MAX_DIMS] = { 0 }; OcSize vsize[OC_TENSOR_MAX_DIMS]; OcIndex vstrides[OC_TENSOR_MAX_DIMS];
   int vnd, d, result = -1; OcModuleCore *m = OcModuleCore_forDevice(tensor->device);
   if (index_view(tensor, indices, &view, &off, vsize, vstrides, &vnd) != 0) return -1;
   if ((v = OcTensor_createFromStorage(tensor->storage, vnd, vsize, vstrides, tensor->offset, tensor->dtype)) == NULL) goto final;
   offsets[0] = off; view.ndims = vnd; view.view = v; view.offsets = offsets;
   if (src->ndims != vnd || src->dtype != tensor->dtype || src->device != tensor->device) { OcErrorMessage("Source of an indexed assignment must match the view"); goto final; }
   for (d = 0; d < vnd; d++) if (src->size[d] != vsize[d]) { OcErrorMessage("Source size mismatch in dimension %d", d); goto final; }
   result = m->Tensor_setIndex(&view, src);
final:
   if (v) OcDecrefTensor(v);
   if (off) OcDecrefTensor(off);
   return result;
}
