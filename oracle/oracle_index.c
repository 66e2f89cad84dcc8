/* TEST INFRASTRUCTURE (see oracle.h).
 * Index operations, restated from solid/src/core/cpu/template_index.c (add_if_negative :257-270,
 * index_to_offset :273-297, get_index :504-511, set_index :517-524, fill_index :530-537) and the walk of
 * solid/include/solid/core/cpu/index.h:54-140: in dimension d the element offset advances by
 * offsets[d][i] when a table is given and by i * strides[d] otherwise. Elements are moved as
 * raw bytes, which is what the typed assignments of the reference amount to.
 * Pinned by tests/test_index_cpu.py against numpy's integer-array indexing.
 */
#include "oracle.h"
#include "oracle_types.h"
#include <string.h>

static const int o_esize[O_NTYPES] = { 1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 4, 8, 16 };

int oracle_add_if_negative(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, och_scalar value)
{
   size_t idx[O_MAX_DIMS] = { 0 }, n = 1, e; int d;
   if (dtype < O_INT8 || dtype > O_INT64 || ndims < 0 || ndims > O_MAX_DIMS) return -1;
   for (d = 0; d < ndims; d++) n *= size[d];
   for (e = 0; e < n; e++)
   {  ptrdiff_t off = 0;
      for (d = 0; d < ndims; d++) off += (ptrdiff_t)idx[d] * strides[d];
      switch (dtype)
      {  case O_INT8:  { int8_t  *p = (int8_t  *)((char *)ptr + off); if (*p < 0) *p = (int8_t)(*p + value._int8); } break;
         case O_INT16: { int16_t *p = (int16_t *)((char *)ptr + off); if (*p < 0) *p = (int16_t)(*p + value._int16); } break;
         case O_INT32: { int32_t *p = (int32_t *)((char *)ptr + off); if (*p < 0) *p = (int32_t)((uint32_t)*p + (uint32_t)value._int32); } break;
         default:      { int64_t *p = (int64_t *)((char *)ptr + off); if (*p < 0) *p = (int64_t)((uint64_t)*p + (uint64_t)value._int64); } break;
      }
      for (d = 0; d < ndims; d++) { if (++idx[d] < size[d]) break; idx[d] = 0; }
   }
   return 0;
}

int oracle_index_to_offset(int dtype, int nstrides, const int64_t *strides, ptrdiff_t stride_reduce, size_t nelem,
                           ptrdiff_t stride1, const void *ptr1, ptrdiff_t stride2, void *ptr2)
{
   size_t j; int i;
   if (dtype < O_UINT8 || dtype > O_INT64) return -1;
   for (j = 0; j < nelem; j++)
   {  int64_t s = 0;
      for (i = 0; i < nstrides; i++)
      {  const char *p = (const char *)ptr1 + (ptrdiff_t)j * stride1 + (ptrdiff_t)i * stride_reduce; int64_t v;
         switch (dtype)
         {  case O_UINT8: v = *(const uint8_t *)p; break;   case O_UINT16: v = *(const uint16_t *)p; break;
            case O_UINT32: v = *(const uint32_t *)p; break; case O_UINT64: v = (int64_t)*(const uint64_t *)p; break;
            case O_INT8: v = *(const int8_t *)p; break;     case O_INT16: v = *(const int16_t *)p; break;
            case O_INT32: v = *(const int32_t *)p; break;   default: v = *(const int64_t *)p; break;
         }
         s = (int64_t)((uint64_t)s + (uint64_t)strides[i] * (uint64_t)v);
      }
      *(int64_t *)((char *)ptr2 + (ptrdiff_t)j * stride2) = s;
   }
   return 0;
}

/* mode 0: gather, 1: scatter, 2: fill */
static int o_index(int mode, int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                   const ptrdiff_t *strides2, void *ptr2, const och_scalar *value)
{
   size_t idx[O_MAX_DIMS] = { 0 }, n = 1, e; int d, es;
   if (dtype < 0 || dtype >= O_NTYPES || ndims < 0 || ndims > O_MAX_DIMS) return -1;
   es = o_esize[dtype];
   for (d = 0; d < ndims; d++) n *= size[d];
   for (e = 0; e < n; e++)
   {  ptrdiff_t o1 = 0, o2 = 0;
      for (d = 0; d < ndims; d++)
      {  o1 += (offsets && offsets[d]) ? (ptrdiff_t)offsets[d][idx[d]] : (ptrdiff_t)idx[d] * strides1[d];
         if (mode != 2) o2 += (ptrdiff_t)idx[d] * strides2[d];
      }
      if (mode == 0) memcpy((char *)ptr2 + o2, (char *)ptr1 + o1, es);
      else if (mode == 1) memcpy((char *)ptr1 + o1, (char *)ptr2 + o2, es);
      else memcpy((char *)ptr1 + o1, value, es);
      for (d = 0; d < ndims; d++) { if (++idx[d] < size[d]) break; idx[d] = 0; }
   }
   return 0;
}
int oracle_get_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                     const ptrdiff_t *strides2, void *ptr2)
{  return o_index(0, dtype, ndims, size, offsets, strides1, ptr1, strides2, ptr2, NULL); }
int oracle_set_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides1, void *ptr1,
                     const ptrdiff_t *strides2, void *ptr2)
{  return o_index(1, dtype, ndims, size, offsets, strides1, ptr1, strides2, ptr2, NULL); }
int oracle_fill_index(int dtype, int ndims, const size_t *size, int64_t **offsets, const ptrdiff_t *strides, void *ptr, och_scalar value)
{  return o_index(2, dtype, ndims, size, offsets, strides, ptr, NULL, NULL, &value); }

/* find / mask-to-offset (template_index.c:296-500): positions of the non-zero elements of a bool tensor in element
   order (dimension 0 fastest). multiplier == NULL: ndims indices per hit; otherwise sum of index * multiplier. */
size_t oracle_find(int ndims, const size_t *size, const ptrdiff_t *strides, const void *ptr, const int64_t *multiplier, int64_t *out)
{
   size_t idx[O_MAX_DIMS] = { 0 }, n = 1, e, count = 0; int d;
   for (d = 0; d < ndims; d++) n *= size[d];
   for (e = 0; e < n; e++)
   {  ptrdiff_t off = 0;
      for (d = 0; d < ndims; d++) off += (ptrdiff_t)idx[d] * strides[d];
      if (((const char *)ptr)[off] != 0)
      {  if (out)
         {  if (multiplier) { int64_t s = 0; for (d = 0; d < ndims; d++) s += (int64_t)idx[d] * multiplier[d]; out[count] = s; }
            else for (d = 0; d < ndims; d++) out[count * ndims + d] = (int64_t)idx[d];
         }
         count++;
      }
      for (d = 0; d < ndims; d++) { if (++idx[d] < size[d]) break; idx[d] = 0; }
   }
   return count;
}
