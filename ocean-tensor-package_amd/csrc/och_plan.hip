/* och_elemwise_analyze: the host-side analysis of an elementwise call (normalisation, kernel
 * choice, chunking) run without a launch. Uses the same routines as the launchers. */
#include "och_elemwise.h"

namespace och {

static uint64_t g_ew_launch_limit = 0;
uint64_t ew_launch_limit() { return g_ew_launch_limit ? g_ew_launch_limit : 0xFFFF0000ull; }

template <int NOPS>
static int analyze(const int *elemsize, int ndims, const size_t *size, const ptrdiff_t *const *strides, void *const *ptrs,
                   och_elemwise_plan *plan)
{
   EwShape<NOPS> shape;
   const ptrdiff_t *st[NOPS]; void *pp[NOPS]; int es[NOPS]; int maxes = 1;
   for (int k = 0; k < NOPS; k++) { st[k] = strides[k]; pp[k] = ptrs[k]; es[k] = elemsize[k]; if (es[k] > maxes) maxes = es[k]; }
   if (ew_normalize<NOPS>(shape, ndims, size, st, pp, NOPS - 1, true) != 0) return -1;
   memset(plan, 0, sizeof(*plan));
   plan->ndims = (shape.nelem == 0) ? 0 : shape.ndims;
   if (shape.nelem == 0) return 0;
   for (int d = 0; d < shape.ndims; d++)
   {  plan->size[d] = shape.size[d];
      for (int k = 0; k < NOPS; k++) plan->strides[k][d] = shape.stride[k][d];
   }
   for (int k = 0; k < NOPS; k++) plan->offset[k] = shape.ptr[k] - (char *)ptrs[k];
   const int vec = (16 / maxes) > 0 ? (16 / maxes) : 1;
   const int (&esr)[NOPS] = es;
   int launches = 0; bool first = true;
   ew_launch_chunked<NOPS>(shape, 0, [&](const EwShape<NOPS> &s, uint64_t flat0) -> int
   {  int kernel = OCH_KERNEL_SINGLE, v = 1, n = 1;
      EwParams<NOPS> p;
      bool tiled = false;
      if (NOPS >= 2)
      {  TileParams<NOPS> tp; dim3 grid; size_t lds; int tb[NOPS];
         const int tile = tile_dim((size_t)maxes);
         for (int k = 0; k < NOPS; k++)
         {  int pad = es[k] >= 4 ? 1 : 4 / es[k];
            tb[k] = (k == NOPS - 1) ? 0 : ((tile * (tile + pad) * es[k]) + 15) / 16 * 16;
         }
         const int (&tbr)[NOPS] = tb;
         tiled = ew_tile_params<NOPS>(tp, s, esr, tile, vec, grid, lds, tbr);
      }
      if (tiled) { kernel = OCH_KERNEL_TILED; v = vec; }
      else if (ew_rows_wanted<NOPS>(s, vec, es) && ew_rows_params<NOPS>(p, s, vec, es, flat0))
      {  kernel = OCH_KERNEL_ROWS; v = vec;
         if (first) { plan->row_units = p.div[0].d; plan->row_elements = (size_t)p.row_n0; }
      }
      else if (ew_params<NOPS>(p, s, vec, es, flat0))
      {  bool all = true;
         for (int k = 0; k < NOPS; k++) all = all && (p.vecmode[k] == 1);
         kernel = all ? OCH_KERNEL_WIDE : OCH_KERNEL_MIXED; v = vec;
      }
      else if (vec > 1 && s.ndims == 1 && s.size[0] > (uint64_t)vec)
      {  EwShape<NOPS> body = s;
         body.size[0] = s.size[0] - s.size[0] % vec; body.nelem = body.size[0];
         ew_params<NOPS>(p, body, vec, es, flat0);
         bool all = true;
         for (int k = 0; k < NOPS; k++) all = all && (p.vecmode[k] == 1);
         kernel = all ? OCH_KERNEL_WIDE : OCH_KERNEL_MIXED; v = vec; n = 2;      /* body + tail */
      }
      else ew_params<NOPS>(p, s, 1, es, flat0);
      if (first)
      {  plan->kernel = kernel; plan->vec = v; first = false;
         if (kernel != OCH_KERNEL_TILED)
            for (int d = 0; d < s.ndims; d++)
            {  plan->div_d[d] = p.div[d].d; plan->div_m[d] = p.div[d].m; plan->div_s1[d] = p.div[d].s1; plan->div_s2[d] = p.div[d].s2; }
      }
      launches += n;
      return 0;
   });
   plan->launches = launches;
   return 0;
}

} /* namespace och */

using namespace och;

extern "C" int och_elemwise_row_unit(unsigned unit, int misalignment, int elemsize, int vec, size_t row_elements,
                                     long long *first, int *lo, int *hi)
{  int64_t e0; const bool any = row_unit_range(unit, misalignment, elemsize, vec, row_elements, e0, *lo, *hi);
   *first = e0;
   return any ? 1 : 0;
}
extern "C" size_t och_elemwise_row_units(size_t row_elements, int elemsize, int vec) { return (size_t)row_units(row_elements, elemsize, vec); }

extern "C" int och_elemwise_analyze(int noperands, const int *elemsize, int ndims, const size_t *size,
                                    const ptrdiff_t *const *strides, void *const *ptrs, och_elemwise_plan *plan)
{
   if (!elemsize || !strides || !ptrs || !plan || (ndims > 0 && !size)) return set_error("elemwise_analyze: null argument");
   for (int k = 0; k < noperands && k < 3; k++)
      if (elemsize[k] != 1 && elemsize[k] != 2 && elemsize[k] != 4 && elemsize[k] != 8 && elemsize[k] != 16)
         return set_error("elemwise_analyze: invalid element size %d", elemsize[k]);
   switch (noperands)
   {  case 1: return analyze<1>(elemsize, ndims, size, strides, ptrs, plan);
      case 2: return analyze<2>(elemsize, ndims, size, strides, ptrs, plan);
      case 3: return analyze<3>(elemsize, ndims, size, strides, ptrs, plan);
   }
   return set_error("elemwise_analyze: %d operands are not supported (1 to 3)", noperands);
}

extern "C" int och_elemwise_set_launch_limit(size_t nelem)
{
   if (nelem != 0 && (nelem < 64 || nelem > 0xFFFF0000ull))
      return och::set_error("och_elemwise_set_launch_limit: the limit must be 0 (default) or between 64 and 0xFFFF0000 elements");
   och::g_ew_launch_limit = nelem;
   return 0;
}
