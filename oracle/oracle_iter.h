/* TEST INFRASTRUCTURE (see oracle_types.h).
 * Strided traversal of up to three operands of equal shape, dimension 0
 * fastest, with the CPU module's work split: a contiguous range of the flat
 * index per thread, the first (nelem % nthreads) threads taking one element
 * more (solid/include/solid/core/cpu/apply_elemwise2.h:130-190,
 * reduce_all.h:183-263). nthreads <= 1 is the serial traversal of
 * apply_elemwise3.h:71-132, which Ocean uses for all three-operand operations
 * (apply_elemwise3.h:36,40 pass 0 threads).
 */
#ifndef ORACLE_ITER_H
#define ORACLE_ITER_H
#include "oracle_types.h"
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct
{  int        ndims, nops;
   size_t     size[O_MAX_DIMS];
   ptrdiff_t  stride[3][O_MAX_DIMS];
   size_t     idx[O_MAX_DIMS];
   char      *p[3];
} o_iter;

static inline size_t o_nelem(int ndims, const size_t *size)
{  size_t n = 1; int i; for (i = 0; i < ndims; i++) n *= size[i]; return n; }

/* position the iterator on flat index `start` */
static inline void o_iter_init(o_iter *it, int nops, int ndims, const size_t *size,
                               const ptrdiff_t *const *strides, void *const *ptrs, size_t start)
{
   int d, k;
   it->ndims = (ndims > 0) ? ndims : 1; it->nops = nops;
   for (k = 0; k < nops; k++) it->p[k] = (char *)ptrs[k];
   if (ndims == 0)
   {  it->size[0] = 1; it->idx[0] = 0;
      for (k = 0; k < nops; k++) it->stride[k][0] = 0;
      return;
   }
   for (d = 0; d < ndims; d++)
   {  it->size[d] = size[d];
      it->idx[d] = size[d] ? (start % size[d]) : 0;
      if (size[d]) start /= size[d];
      for (k = 0; k < nops; k++)
      {  it->stride[k][d] = strides[k][d];
         it->p[k] += (ptrdiff_t)it->idx[d] * strides[k][d];
      }
   }
}

/* after `run` elements along dimension 0 were consumed: carry into higher dimensions */
static inline void o_iter_carry(o_iter *it, size_t run)
{
   int d = 0, k;
   it->idx[0] += run;
   for (k = 0; k < it->nops; k++) it->p[k] += (ptrdiff_t)run * it->stride[k][0];
   while (d < it->ndims - 1 && it->idx[d] == it->size[d])
   {  for (k = 0; k < it->nops; k++)
         it->p[k] += it->stride[k][d + 1] - (ptrdiff_t)it->size[d] * it->stride[k][d];
      it->idx[d] = 0; d++; it->idx[d]++;
   }
}

/* range of flat indices of thread `rank` out of `nthreads` */
static inline void o_thread_range(size_t nelem, int rank, int nthreads, size_t *start, size_t *stop)
{
   size_t rem = nelem % (size_t)nthreads, n = nelem / (size_t)nthreads, off;
   if ((size_t)rank < rem) { n++; off = (size_t)rank * n; }
   else off = rem + (size_t)rank * n;
   *start = off; *stop = off + n;
}

/* Loop over flat indices [START, STOP); BODY sees char pointers q0, q1, q2 */
#define O_RANGE_LOOP(NOPS, NDIMS, SIZE, STRIDES, PTRS, START, STOP, ...)                \
   {  o_iter _it; size_t _i = (START), _stop = (STOP);                                  \
      if (_i < _stop)                                                                   \
      {  o_iter_init(&_it, NOPS, NDIMS, SIZE, STRIDES, PTRS, _i);                        \
         while (_i < _stop)                                                             \
         {  size_t _run = _it.size[0] - _it.idx[0], _k;                                 \
            char *q0 = _it.p[0], *q1 = (NOPS > 1) ? _it.p[1] : 0, *q2 = (NOPS > 2) ? _it.p[2] : 0; \
            ptrdiff_t _s0 = _it.stride[0][0], _s1 = (NOPS > 1) ? _it.stride[1][0] : 0,  \
                      _s2 = (NOPS > 2) ? _it.stride[2][0] : 0;                          \
            if (_run > _stop - _i) _run = _stop - _i;                                   \
            for (_k = 0; _k < _run; _k++)                                               \
            {  __VA_ARGS__                                                              \
               q0 += _s0; q1 += _s1; q2 += _s2;                                         \
            }                                                                           \
            (void)q1; (void)q2;                                                         \
            _i += _run; o_iter_carry(&_it, _run);                                       \
         }                                                                              \
      }                                                                                 \
   }

/* Full traversal, serial or split over `NTHREADS` threads */
#define O_ELEMWISE_LOOP(NOPS, NDIMS, SIZE, STRIDES, PTRS, NTHREADS, ...)                \
   {  size_t _nelem = o_nelem(NDIMS, SIZE); int _nt = (NTHREADS);                       \
      if ((size_t)_nt > _nelem) _nt = (int)_nelem;                                      \
      if (_nt <= 1) O_RANGE_LOOP(NOPS, NDIMS, SIZE, STRIDES, PTRS, 0, _nelem, __VA_ARGS__)     \
      else                                                                              \
      {  _Pragma("omp parallel num_threads(_nt)")                                       \
         {  size_t _a, _b;                                                              \
            o_thread_range(_nelem, omp_get_thread_num(), omp_get_num_threads(), &_a, &_b); \
            O_RANGE_LOOP(NOPS, NDIMS, SIZE, STRIDES, PTRS, _a, _b, __VA_ARGS__)             \
         }                                                                              \
      }                                                                                 \
   }

#endif
