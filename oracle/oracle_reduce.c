/* TEST INFRASTRUCTURE (see oracle.h).
 * Full and axis reductions of the CPU oracle.
 *
 * Full reductions reproduce the CPU module's work split (solid/include/solid/core/cpu/
 * reduce_all.h:59-100): with T threads available, T is lowered to nelem/512 when the tensor
 * has fewer than 512*T elements; each thread folds a contiguous range of the flat index
 * (first nelem%T threads one element more) into its own accumulator, the accumulators are
 * combined in thread order, then finalized (sqrt / pow for norms) and converted to the
 * result type. Float sums are therefore folded serially in the input's work precision and
 * depend on the thread count, exactly like Ocean's CPU results do.
 *
 * Axis reductions fold the reduced dimensions serially for each output element, reduced
 * dimension 0 fastest (solid/include/solid/core/cpu/reduce_axis.h, "single" variant; the
 * OpenMP variants change only which thread computes which output, except omp2, which is
 * selected for fewer than 4*T outputs and splits each reduction like a full reduction).
 */
#include "oracle.h"
#include "oracle_convert.h"
#include "oracle_iter.h"

typedef struct { och_scalar b1, b2; double p; } o_red_param;
typedef struct
{  size_t acc_size;
   void (*accumulate)(int, const size_t *, const ptrdiff_t *, void *, size_t, size_t, const o_red_param *, void *);
   void (*combine)(void *, const void *);
   void (*finalize)(void *, const o_red_param *, void *);
} o_red_desc;

#define O_TMPL_FILE "oracle_reduce_tmpl.h"
#include "oracle_foreach_type.h"
#undef O_TMPL_FILE

#define D(op, t) &o_red_##op##_##t##_desc
#define ROW_ALL(op) { D(op, bool), D(op, uint8), D(op, uint16), D(op, uint32), D(op, uint64), D(op, int8), D(op, int16), D(op, int32), \
                      D(op, int64), D(op, half), D(op, float), D(op, double), D(op, chalf), D(op, cfloat), D(op, cdouble) }
#define ROW_FC(op)  { 0, 0, 0, 0, 0, 0, 0, 0, 0, D(op, half), D(op, float), D(op, double), D(op, chalf), D(op, cfloat), D(op, cdouble) }
/* the *_nan variants of integer types are the plain operations (template_reduce_all.c forwards) */
#define ROW_NAN(op, plain) { D(plain, bool), D(plain, uint8), D(plain, uint16), D(plain, uint32), D(plain, uint64), D(plain, int8), \
                      D(plain, int16), D(plain, int32), D(plain, int64), D(op, half), D(op, float), D(op, double), D(op, chalf), D(op, cfloat), D(op, cdouble) }

static const o_red_desc *const o_red_table[OCH_REDUCE_COUNT][O_NTYPES] = {
   [OCH_R_ANY] = ROW_ALL(any), [OCH_R_ALL] = ROW_ALL(all),
   [OCH_R_ALL_FINITE] = ROW_FC(all_finite), [OCH_R_ANY_INF] = ROW_FC(any_inf), [OCH_R_ANY_NAN] = ROW_FC(any_nan),
   [OCH_R_NNZ] = ROW_ALL(nnz), [OCH_R_NNZ_NAN] = ROW_NAN(nnz_nan, nnz),
   [OCH_R_ALL_LT] = ROW_ALL(all_lt), [OCH_R_ALL_LE] = ROW_ALL(all_le), [OCH_R_ALL_GT] = ROW_ALL(all_gt), [OCH_R_ALL_GE] = ROW_ALL(all_ge),
   [OCH_R_ALL_GTLT] = ROW_ALL(all_gtlt), [OCH_R_ALL_GTLE] = ROW_ALL(all_gtle), [OCH_R_ALL_GELT] = ROW_ALL(all_gelt), [OCH_R_ALL_GELE] = ROW_ALL(all_gele),
   [OCH_R_SUM] = ROW_ALL(sum), [OCH_R_SUM_NAN] = ROW_NAN(sum_nan, sum), [OCH_R_PROD] = ROW_ALL(prod), [OCH_R_PROD_NAN] = ROW_NAN(prod_nan, prod),
   [OCH_R_SUM_ABS] = ROW_ALL(sum_abs), [OCH_R_SUM_ABS_NAN] = ROW_NAN(sum_abs_nan, sum_abs),
   [OCH_R_MAXIMUM] = ROW_ALL(maximum), [OCH_R_MINIMUM] = ROW_ALL(minimum),
   [OCH_R_MAXIMUM_ABS] = ROW_ALL(maximum_abs), [OCH_R_MINIMUM_ABS] = ROW_ALL(minimum_abs),
   [OCH_R_NORM] = ROW_ALL(norm), [OCH_R_NORM_NAN] = ROW_NAN(norm_nan, norm),
   [OCH_R_NORM2] = ROW_ALL(norm2), [OCH_R_NORM2_NAN] = ROW_NAN(norm2_nan, norm2),
};

int oracle_reduce_supported(int op, int dtype)
{  return op >= 0 && op < OCH_REDUCE_COUNT && dtype >= 0 && dtype < O_NTYPES && o_red_table[op][dtype] != 0; }

/* result types of reduce_ops.h: logical -> bool; nnz -> uint64; sum/prod -> uint64 | int64 | same;
   sum_abs -> uint64 | magnitude type; max/min -> same; max/min abs -> magnitude type (unsigned twin
   for signed integers); norms -> double for integers and bool, magnitude type otherwise */
int oracle_reduce_result_dtype(int op, int dtype)
{
   int isbool = (dtype == O_BOOL), isuint = (dtype >= O_UINT8 && dtype <= O_UINT64), issint = (dtype >= O_INT8 && dtype <= O_INT64);
   int mag = (dtype >= O_CHALF) ? dtype - 3 : (issint ? dtype - 4 : dtype);
   if (!oracle_reduce_supported(op, dtype)) return -1;
   if (op <= OCH_R_ANY_NAN || (op >= OCH_R_ALL_LT && op <= OCH_R_ALL_GELE)) return O_BOOL;
   if (op == OCH_R_NNZ || op == OCH_R_NNZ_NAN) return O_UINT64;
   if (op >= OCH_R_SUM && op <= OCH_R_PROD_NAN) return (isbool || isuint) ? O_UINT64 : (issint ? O_INT64 : dtype);
   if (op == OCH_R_SUM_ABS || op == OCH_R_SUM_ABS_NAN) return (isbool || isuint || issint) ? O_UINT64 : mag;
   if (op == OCH_R_MAXIMUM || op == OCH_R_MINIMUM) return dtype;
   if (op == OCH_R_MAXIMUM_ABS || op == OCH_R_MINIMUM_ABS) return mag;
   return (isbool || isuint || issint) ? O_DOUBLE : mag;
}

#define O_MAX_THREADS 1024

int oracle_reduce_all(int op, int dtype, int ndims, const size_t *size, const ptrdiff_t *strides,
                void *ptr, const och_scalar *param1, const och_scalar *param2, double p,
                void *result, int nthreads)
{
   const o_red_desc *d;
   o_red_param prm;
   size_t nelem = o_nelem(ndims, size);
   if (!oracle_reduce_supported(op, dtype)) return -1;
   d = o_red_table[op][dtype];
   memset(&prm, 0, sizeof(prm));
   if (param1) prm.b1 = *param1;
   if (param2) prm.b2 = *param2;
   prm.p = p;
   if (nthreads > O_MAX_THREADS) nthreads = O_MAX_THREADS;
   if (nthreads < 1) nthreads = 1;
   if (nelem < (size_t)nthreads * 512) nthreads = (int)(nelem / 512);
   if (nthreads > 1)
   {  static char partial[O_MAX_THREADS][32];
      int j;
      #pragma omp parallel num_threads(nthreads)
      {  size_t a, b; int rank = 0, nt = 1;
#ifdef _OPENMP
         rank = omp_get_thread_num(); nt = omp_get_num_threads();
#endif
         o_thread_range(nelem, rank, nt, &a, &b);
         d->accumulate(ndims, size, strides, ptr, a, b, &prm, partial[rank]);
      }
      for (j = 1; j < nthreads; j++) d->combine(partial[0], partial[j]);
      d->finalize(partial[0], &prm, result);
   }
   else
   {  char acc[32];
      d->accumulate(ndims, size, strides, ptr, 0, nelem, &prm, acc);
      d->finalize(acc, &prm, result);
   }
   return 0;
}

int oracle_reduce_axis(int op, int dtype, const och_reduce_axis_config *c, double p)
{
   const o_red_desc *d;
   o_red_param prm;
   size_t nout, relem, i;
   o_iter it;
   const ptrdiff_t *st[2] = { c->strides1, c->strides2 };
   void *pp[2] = { c->ptr1, c->ptr2 };
   if (!oracle_reduce_supported(op, dtype)) return -1;
   d = o_red_table[op][dtype];
   memset(&prm, 0, sizeof(prm));
   prm.p = p;
   nout = o_nelem(c->ndims, c->size);
   relem = o_nelem(c->rdims, c->rsize);
   if (nout == 0) return 0;
   o_iter_init(&it, 2, c->ndims, c->size, st, pp, 0);
   for (i = 0; i < nout; i++)
   {  char acc[32];
      d->accumulate(c->rdims, c->rsize, c->rstrides, it.p[0], 0, relem, &prm, acc);
      d->finalize(acc, &prm, it.p[1]);
      o_iter_carry(&it, 1);
   }
   return 0;
}

/* The same axis reduction with the CPU module's multi-thread split for many outputs (reduce_axis.h:65-104, 300-400,
   variant "omp1"): the outputs are dealt to the threads in contiguous ranges of the flat output index and every
   thread reduces its outputs on its own, so the result equals the serial one bit for bit. Fewer than 4 outputs per
   thread, or 256 operations or fewer, run serially here (the reference's cooperative variant "omp2" reorders the
   additions of one output; it is not restated). */
int oracle_reduce_axis_threads(int op, int dtype, const och_reduce_axis_config *c, double p, int nthreads)
{
   const o_red_desc *d;
   o_red_param prm;
   size_t nout, relem;
   const ptrdiff_t *st[2] = { c->strides1, c->strides2 };
   void *pp[2] = { c->ptr1, c->ptr2 };
   if (!oracle_reduce_supported(op, dtype)) return -1;
   nout = o_nelem(c->ndims, c->size);
   relem = o_nelem(c->rdims, c->rsize);
   if (nthreads <= 1 || nout * relem <= 256 || nout < 4 * (size_t)nthreads) return oracle_reduce_axis(op, dtype, c, p);
   d = o_red_table[op][dtype];
   memset(&prm, 0, sizeof(prm));
   prm.p = p;
   #pragma omp parallel num_threads(nthreads)
   {  size_t a, b, i; int rank = 0, nt = 1;
      o_iter it;
#ifdef _OPENMP
      rank = omp_get_thread_num(); nt = omp_get_num_threads();
#endif
      o_thread_range(nout, rank, nt, &a, &b);
      if (a < b)
      {  o_iter_init(&it, 2, c->ndims, c->size, st, pp, a);
         for (i = a; i < b; i++)
         {  char acc[32];
            d->accumulate(c->rdims, c->rsize, c->rstrides, it.p[0], 0, relem, &prm, acc);
            d->finalize(acc, &prm, it.p[1]);
            o_iter_carry(&it, 1);
         }
      }
   }
   return 0;
}
