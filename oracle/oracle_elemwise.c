/* TEST INFRASTRUCTURE (see oracle.h).
 * Elementwise part of the CPU oracle: binary and unary operations for all 15
 * element types, converting copies, byte swapping, fill and steps.
 * Follows solid/src/core/cpu/template_{binary,unary,copy,byteswap,fill,steps}.c
 * and the loop/threading macros solid/include/solid/core/cpu/apply_elemwise{1,2,2b,3}.h.
 * parity: every per-element function is pinned against the reference's own operation
 * macros (oracle/_ref, tests/test_oracle_ref.py) except where that file says otherwise.
 */
#include "oracle.h"
#include "oracle_convert.h"
#include "oracle_iter.h"

int oracle_max_threads(void)
{
#ifdef _OPENMP
   return omp_get_max_threads();
#else
   return 1;
#endif
}

float    oracle_half_to_float(uint16_t h) { return o_half_to_float(h); }
uint16_t oracle_float_to_half(float f)    { return o_float_to_half(f); }

/* ---- instantiate the per-type operation loops ----------------------------- */
#define O_TMPL_FILE "oracle_ops_tmpl.h"
#include "oracle_foreach_type.h"
#undef O_TMPL_FILE

/* ---- tables ------------------------------------------------------------------ */
typedef int (*o_bin_fn)(int, const size_t *, const ptrdiff_t *, void *, const ptrdiff_t *, void *, const ptrdiff_t *, void *);
typedef int (*o_un_fn)(int, const size_t *, const ptrdiff_t *, void *, const ptrdiff_t *, void *, int);

#define ROW_ALL(P, N)  { P##N##_bool, P##N##_uint8, P##N##_uint16, P##N##_uint32, P##N##_uint64, P##N##_int8, P##N##_int16, \
                         P##N##_int32, P##N##_int64, P##N##_half, P##N##_float, P##N##_double, P##N##_chalf, P##N##_cfloat, P##N##_cdouble }
#define ROW_NB(P, N)   { 0, P##N##_uint8, P##N##_uint16, P##N##_uint32, P##N##_uint64, P##N##_int8, P##N##_int16, \
                         P##N##_int32, P##N##_int64, P##N##_half, P##N##_float, P##N##_double, P##N##_chalf, P##N##_cfloat, P##N##_cdouble }

/* Aliases of template_binary.c:143-178: bool min/max/fmin/fmax are and/or; integer fmin/fmax are
   min/max; divide of non-signed types is true_divide; floor_divide of bool/unsigned is
   true_divide and their fmod is mod; bool bitwise ops are the logical ones. */
static const o_bin_fn o_binary_table[OCH_BINARY_COUNT][O_NTYPES] = {
   [OCH_ADD]         = ROW_ALL(o_bin_, add),
   [OCH_SUBTRACT]    = ROW_ALL(o_bin_, subtract),
   [OCH_MULTIPLY]    = ROW_ALL(o_bin_, multiply),
   [OCH_TRUE_DIVIDE] = ROW_ALL(o_bin_, true_divide),
   [OCH_DIVIDE]      = { o_bin_true_divide_bool, o_bin_true_divide_uint8, o_bin_true_divide_uint16, o_bin_true_divide_uint32,
                         o_bin_true_divide_uint64, o_bin_divide_int8, o_bin_divide_int16, o_bin_divide_int32, o_bin_divide_int64,
                         o_bin_true_divide_half, o_bin_true_divide_float, o_bin_true_divide_double,
                         o_bin_true_divide_chalf, o_bin_true_divide_cfloat, o_bin_true_divide_cdouble },
   [OCH_FLOOR_DIVIDE]= { o_bin_true_divide_bool, o_bin_true_divide_uint8, o_bin_true_divide_uint16, o_bin_true_divide_uint32,
                         o_bin_true_divide_uint64, o_bin_floor_divide_int8, o_bin_floor_divide_int16, o_bin_floor_divide_int32,
                         o_bin_floor_divide_int64, o_bin_floor_divide_half, o_bin_floor_divide_float, o_bin_floor_divide_double, 0, 0, 0 },
   [OCH_POWER]       = ROW_ALL(o_bin_, power),
   [OCH_MOD]         = { o_bin_mod_bool, o_bin_mod_uint8, o_bin_mod_uint16, o_bin_mod_uint32, o_bin_mod_uint64, o_bin_mod_int8,
                         o_bin_mod_int16, o_bin_mod_int32, o_bin_mod_int64, o_bin_mod_half, o_bin_mod_float, o_bin_mod_double, 0, 0, 0 },
   [OCH_FMOD]        = { o_bin_mod_bool, o_bin_mod_uint8, o_bin_mod_uint16, o_bin_mod_uint32, o_bin_mod_uint64, o_bin_fmod_int8,
                         o_bin_fmod_int16, o_bin_fmod_int32, o_bin_fmod_int64, o_bin_fmod_half, o_bin_fmod_float, o_bin_fmod_double, 0, 0, 0 },
   [OCH_MIN]         = { o_bin_bitwise_and_bool, o_bin_min_uint8, o_bin_min_uint16, o_bin_min_uint32, o_bin_min_uint64, o_bin_min_int8,
                         o_bin_min_int16, o_bin_min_int32, o_bin_min_int64, o_bin_min_half, o_bin_min_float, o_bin_min_double,
                         o_bin_min_chalf, o_bin_min_cfloat, o_bin_min_cdouble },
   [OCH_MAX]         = { o_bin_bitwise_or_bool, o_bin_max_uint8, o_bin_max_uint16, o_bin_max_uint32, o_bin_max_uint64, o_bin_max_int8,
                         o_bin_max_int16, o_bin_max_int32, o_bin_max_int64, o_bin_max_half, o_bin_max_float, o_bin_max_double,
                         o_bin_max_chalf, o_bin_max_cfloat, o_bin_max_cdouble },
   [OCH_FMIN]        = { o_bin_bitwise_and_bool, o_bin_min_uint8, o_bin_min_uint16, o_bin_min_uint32, o_bin_min_uint64, o_bin_min_int8,
                         o_bin_min_int16, o_bin_min_int32, o_bin_min_int64, o_bin_fmin_half, o_bin_fmin_float, o_bin_fmin_double,
                         o_bin_fmin_chalf, o_bin_fmin_cfloat, o_bin_fmin_cdouble },
   [OCH_FMAX]        = { o_bin_bitwise_or_bool, o_bin_max_uint8, o_bin_max_uint16, o_bin_max_uint32, o_bin_max_uint64, o_bin_max_int8,
                         o_bin_max_int16, o_bin_max_int32, o_bin_max_int64, o_bin_fmax_half, o_bin_fmax_float, o_bin_fmax_double,
                         o_bin_fmax_chalf, o_bin_fmax_cfloat, o_bin_fmax_cdouble },
   [OCH_LT] = ROW_ALL(o_bin_, lt), [OCH_LE] = ROW_ALL(o_bin_, le), [OCH_EQ] = ROW_ALL(o_bin_, eq),
   [OCH_NE] = ROW_ALL(o_bin_, ne), [OCH_GE] = ROW_ALL(o_bin_, ge), [OCH_GT] = ROW_ALL(o_bin_, gt),
#define ROW_INTB(N) { o_bin_##N##_bool, o_bin_##N##_uint8, o_bin_##N##_uint16, o_bin_##N##_uint32, o_bin_##N##_uint64, \
                      o_bin_##N##_int8, o_bin_##N##_int16, o_bin_##N##_int32, o_bin_##N##_int64, 0, 0, 0, 0, 0, 0 }
   [OCH_BITWISE_AND] = ROW_INTB(bitwise_and), [OCH_BITWISE_OR] = ROW_INTB(bitwise_or), [OCH_BITWISE_XOR] = ROW_INTB(bitwise_xor),
   [OCH_LOGICAL_AND] = { o_bin_bitwise_and_bool }, [OCH_LOGICAL_OR] = { o_bin_bitwise_or_bool }, [OCH_LOGICAL_XOR] = { o_bin_bitwise_xor_bool },
   [OCH_BITSHIFT_LEFT] = ROW_INTB(bitshift_left), [OCH_BITSHIFT_RIGHT] = ROW_INTB(bitshift_right),
};

#define ROW_FC(N)   { 0, 0, 0, 0, 0, 0, 0, 0, 0, o_un_##N##_half, o_un_##N##_float, o_un_##N##_double, o_un_##N##_chalf, o_un_##N##_cfloat, o_un_##N##_cdouble }
#define ROW_NC(N)   { o_un_##N##_bool, o_un_##N##_uint8, o_un_##N##_uint16, o_un_##N##_uint32, o_un_##N##_uint64, o_un_##N##_int8, \
                      o_un_##N##_int16, o_un_##N##_int32, o_un_##N##_int64, o_un_##N##_half, o_un_##N##_float, o_un_##N##_double, 0, 0, 0 }
/* Aliases of template_unary.c:128-140: bool negative and bitwise_not are logical_not; absolute of
   non-complex types is fabs. */
static const o_un_fn o_unary_table[OCH_UNARY_COUNT][O_NTYPES] = {
   [OCH_NEGATIVE]    = { o_un_logical_not_bool, 0, 0, 0, 0, o_un_negative_int8, o_un_negative_int16, o_un_negative_int32, o_un_negative_int64,
                         o_un_negative_half, o_un_negative_float, o_un_negative_double, o_un_negative_chalf, o_un_negative_cfloat, o_un_negative_cdouble },
   [OCH_BITWISE_NOT] = { o_un_logical_not_bool, o_un_bitwise_not_uint8, o_un_bitwise_not_uint16, o_un_bitwise_not_uint32, o_un_bitwise_not_uint64,
                         o_un_bitwise_not_int8, o_un_bitwise_not_int16, o_un_bitwise_not_int32, o_un_bitwise_not_int64, 0, 0, 0, 0, 0, 0 },
   [OCH_LOGICAL_NOT] = { o_un_logical_not_bool },
   [OCH_CONJ]        = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, o_un_conj_chalf, o_un_conj_cfloat, o_un_conj_cdouble },
   [OCH_RECIPROCAL] = ROW_NB(o_un_, reciprocal),
   [OCH_SIN] = ROW_NB(o_un_, sin), [OCH_COS] = ROW_NB(o_un_, cos), [OCH_TAN] = ROW_NB(o_un_, tan),
   [OCH_SINH] = ROW_NB(o_un_, sinh), [OCH_COSH] = ROW_NB(o_un_, cosh), [OCH_TANH] = ROW_NB(o_un_, tanh),
   [OCH_ARCSIN] = ROW_NB(o_un_, arcsin), [OCH_ARCCOS] = ROW_NB(o_un_, arccos), [OCH_ARCTAN] = ROW_NB(o_un_, arctan),
   [OCH_ARCSINH] = ROW_NB(o_un_, arcsinh), [OCH_ARCCOSH] = ROW_NB(o_un_, arccosh), [OCH_ARCTANH] = ROW_NB(o_un_, arctanh),
   [OCH_SQRT] = ROW_NB(o_un_, sqrt), [OCH_CBRT] = ROW_NB(o_un_, cbrt), [OCH_SQUARE] = ROW_NB(o_un_, square),
   [OCH_EXP] = ROW_NB(o_un_, exp), [OCH_EXP2] = ROW_NB(o_un_, exp2), [OCH_EXP10] = ROW_NB(o_un_, exp10), [OCH_EXPM1] = ROW_NB(o_un_, expm1),
   [OCH_LOG] = ROW_NB(o_un_, log), [OCH_LOG2] = ROW_NB(o_un_, log2), [OCH_LOG10] = ROW_NB(o_un_, log10), [OCH_LOG1P] = ROW_NB(o_un_, log1p),
   [OCH_ABSOLUTE]    = { o_un_fabs_bool, o_un_fabs_uint8, o_un_fabs_uint16, o_un_fabs_uint32, o_un_fabs_uint64, o_un_fabs_int8, o_un_fabs_int16,
                         o_un_fabs_int32, o_un_fabs_int64, o_un_fabs_half, o_un_fabs_float, o_un_fabs_double,
                         o_un_absolute_chalf, o_un_absolute_cfloat, o_un_absolute_cdouble },
   [OCH_FABS] = ROW_ALL(o_un_, fabs), [OCH_SIGN] = ROW_ALL(o_un_, sign),
   [OCH_CEIL] = ROW_FC(ceil), [OCH_FLOOR] = ROW_FC(floor), [OCH_TRUNC] = ROW_FC(trunc), [OCH_ROUND] = ROW_FC(round),
   [OCH_ISINF] = ROW_ALL(o_un_, isinf), [OCH_ISNAN] = ROW_ALL(o_un_, isnan), [OCH_ISFINITE] = ROW_ALL(o_un_, isfinite),
   [OCH_ISPOSINF] = ROW_NC(isposinf), [OCH_ISNEGINF] = ROW_NC(isneginf),
};

int oracle_binary_supported(int op, int dtype)
{  return op >= 0 && op < OCH_BINARY_COUNT && dtype >= 0 && dtype < O_NTYPES && o_binary_table[op][dtype] != 0; }
int oracle_unary_supported(int op, int dtype)
{  return op >= 0 && op < OCH_UNARY_COUNT && dtype >= 0 && dtype < O_NTYPES && o_unary_table[op][dtype] != 0; }

int oracle_binary(int op, int dtype, int ndims, const size_t *size,
                  const ptrdiff_t *s1, void *p1, const ptrdiff_t *s2, void *p2, const ptrdiff_t *s3, void *p3)
{
   if (!oracle_binary_supported(op, dtype)) return -1;
   if (p3 == 0 && s3 == 0) { p3 = p1; s3 = s1; }
   return o_binary_table[op][dtype](ndims, size, s1, p1, s2, p2, s3, p3);
}

int oracle_unary(int op, int dtype, int ndims, const size_t *size,
                 const ptrdiff_t *s1, void *p1, const ptrdiff_t *s2, void *p2, int nthreads)
{
   if (!oracle_unary_supported(op, dtype)) return -1;
   if (p2 == 0 && s2 == 0) { p2 = p1; s2 = s1; }
   return o_unary_table[op][dtype](ndims, size, s1, p1, s2, p2, nthreads);
}

/* ---- SOLID_ASSIGN between any two types, on pointers ------------------------ */
typedef void (*o_assign_fn)(const void *src, void *dst);

#define O_DEF_ASSIGN_RR(S, D) \
   static void o_assign_##S##_##D(const void *s, void *d) { *(o_t_##D *)d = o_cvt_##S##_##D(*(const o_t_##S *)s); }
#define O_ROW_RR(A, S) O_REAL_TYPES_INNER(O_SWAP_RR, S)
#define O_SWAP_RR(S, D) O_DEF_ASSIGN_RR(S, D)
O_REAL_TYPES(O_ROW_RR, _)

/* real S -> complex with part type P; complex with part P -> real D; complex -> complex */
#define O_COMPLEX_PARTS(M, A) M(A, chalf, half) M(A, cfloat, float) M(A, cdouble, double)
#define O_COMPLEX_PARTS_INNER(M, A) M(A, chalf, half) M(A, cfloat, float) M(A, cdouble, double)
#define O_DEF_ASSIGN_RC(S, C, P) \
   static void o_assign_##S##_##C(const void *s, void *d) \
   {  o_t_##C *z = (o_t_##C *)d; z->real = o_cvt_##S##_##P(*(const o_t_##S *)s); z->imag = o_cvt_uint8_##P(0); }
#define O_ROW_RC(A, S) O_COMPLEX_PARTS(O_SWAP_RC, S)
#define O_SWAP_RC(S, C, P) O_DEF_ASSIGN_RC(S, C, P)
O_REAL_TYPES(O_ROW_RC, _)

#define O_DEF_ASSIGN_CR_bool(C, P) \
   static void o_assign_##C##_bool(const void *s, void *d) \
   {  const o_t_##C *x = (const o_t_##C *)s; *(o_bool *)d = (o_cvt_##P##_bool(x->real) || o_cvt_##P##_bool(x->imag)) ? 1 : 0; }
#define O_DEF_ASSIGN_CR(C, P, D) \
   static void o_assign_##C##_##D(const void *s, void *d) { *(o_t_##D *)d = o_cvt_##P##_##D(((const o_t_##C *)s)->real); }
#define O_CR_ALL(C, P) O_DEF_ASSIGN_CR_bool(C, P) \
   O_DEF_ASSIGN_CR(C, P, uint8) O_DEF_ASSIGN_CR(C, P, uint16) O_DEF_ASSIGN_CR(C, P, uint32) O_DEF_ASSIGN_CR(C, P, uint64) \
   O_DEF_ASSIGN_CR(C, P, int8) O_DEF_ASSIGN_CR(C, P, int16) O_DEF_ASSIGN_CR(C, P, int32) O_DEF_ASSIGN_CR(C, P, int64) \
   O_DEF_ASSIGN_CR(C, P, half) O_DEF_ASSIGN_CR(C, P, float) O_DEF_ASSIGN_CR(C, P, double)
O_CR_ALL(chalf, half) O_CR_ALL(cfloat, float) O_CR_ALL(cdouble, double)

#define O_DEF_ASSIGN_CC(C1, P1, C2, P2) \
   static void o_assign_##C1##_##C2(const void *s, void *d) \
   {  const o_t_##C1 *x = (const o_t_##C1 *)s; o_t_##C2 *z = (o_t_##C2 *)d; \
      z->real = o_cvt_##P1##_##P2(x->real); z->imag = o_cvt_##P1##_##P2(x->imag); }
#define O_CC_ROW(C1, P1) O_DEF_ASSIGN_CC(C1, P1, chalf, half) O_DEF_ASSIGN_CC(C1, P1, cfloat, float) O_DEF_ASSIGN_CC(C1, P1, cdouble, double)
O_CC_ROW(chalf, half) O_CC_ROW(cfloat, float) O_CC_ROW(cdouble, double)

#define O_ASSIGN_ROW(S) { o_assign_##S##_bool, o_assign_##S##_uint8, o_assign_##S##_uint16, o_assign_##S##_uint32, o_assign_##S##_uint64, \
   o_assign_##S##_int8, o_assign_##S##_int16, o_assign_##S##_int32, o_assign_##S##_int64, o_assign_##S##_half, o_assign_##S##_float, \
   o_assign_##S##_double, o_assign_##S##_chalf, o_assign_##S##_cfloat, o_assign_##S##_cdouble }
static const o_assign_fn o_assign_table[O_NTYPES][O_NTYPES] = {
   O_ASSIGN_ROW(bool), O_ASSIGN_ROW(uint8), O_ASSIGN_ROW(uint16), O_ASSIGN_ROW(uint32), O_ASSIGN_ROW(uint64),
   O_ASSIGN_ROW(int8), O_ASSIGN_ROW(int16), O_ASSIGN_ROW(int32), O_ASSIGN_ROW(int64),
   O_ASSIGN_ROW(half), O_ASSIGN_ROW(float), O_ASSIGN_ROW(double), O_ASSIGN_ROW(chalf), O_ASSIGN_ROW(cfloat), O_ASSIGN_ROW(cdouble)
};

/* Copy between tensors of equal element count whose shapes may differ: each side is walked
   in its own dimension order, dimension 0 fastest (apply_elemwise2b.h). When swap is set the
   source element is byte-reversed part by part before it is converted
   (SOLID_BYTESWAP_ASSIGN, dtype_assign.h:297-371). */
static int o_copy_generic(int ts, int td, int swap,
                          int nd1, const size_t *size1, const ptrdiff_t *st1, void *p1,
                          int nd2, const size_t *size2, const ptrdiff_t *st2, void *p2, int nthreads)
{
   size_t nelem = o_nelem(nd1, size1);
   o_assign_fn fn;
   if (ts < 0 || ts >= O_NTYPES || td < 0 || td >= O_NTYPES) return -1;
   if (nelem != o_nelem(nd2, size2)) return -1;
   fn = o_assign_table[ts][td];
   if (nthreads < 1) nthreads = 1;
   if ((size_t)nthreads > nelem) nthreads = (int)(nelem ? nelem : 1);
   #pragma omp parallel num_threads(nthreads)
   {
      size_t a, b, i;
      o_iter it1, it2;
      const ptrdiff_t *sa[1] = { st1 }, *sb[1] = { st2 };
      void *pa[1] = { p1 }, *pb[1] = { p2 };
      int rank = 0, nt = 1;
#ifdef _OPENMP
      rank = omp_get_thread_num(); nt = omp_get_num_threads();
#endif
      o_thread_range(nelem, rank, nt, &a, &b);
      if (a < b)
      {  o_iter_init(&it1, 1, nd1, size1, sa, pa, a);
         o_iter_init(&it2, 1, nd2, size2, sb, pb, a);
         for (i = a; i < b; i++)
         {  if (swap)
            {  o_cdouble tmp;
               o_swap_parts(it1.p[0], &tmp, o_part_size[ts], o_part_count[ts]);
               fn(&tmp, it2.p[0]);
            }
            else fn(it1.p[0], it2.p[0]);
            o_iter_carry(&it1, 1); o_iter_carry(&it2, 1);
         }
      }
   }
   return 0;
}

int oracle_copy(int ts, int td, int nd1, const size_t *size1, const ptrdiff_t *st1, void *p1,
                int nd2, const size_t *size2, const ptrdiff_t *st2, void *p2, int nthreads)
{  return o_copy_generic(ts, td, 0, nd1, size1, st1, p1, nd2, size2, st2, p2, nthreads); }

int oracle_byteswap_copy(int ts, int td, int nd1, const size_t *size1, const ptrdiff_t *st1, void *p1,
                int nd2, const size_t *size2, const ptrdiff_t *st2, void *p2, int nthreads)
{  return o_copy_generic(ts, td, 1, nd1, size1, st1, p1, nd2, size2, st2, p2, nthreads); }

int oracle_byteswap(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, int nthreads)
{
   const ptrdiff_t *st[1] = { strides }; void *pp[1] = { ptr };
   int w, n;
   if (dtype < 0 || dtype >= O_NTYPES) return -1;
   w = o_part_size[dtype]; n = o_part_count[dtype];
   O_ELEMWISE_LOOP(1, ndims, size, st, pp, nthreads, { o_swap_parts(q0, q0, w, n); })
   return 0;
}

/* ---- fill, fill_nan, masked_fill (template_fill.c) ------------------------- */
int oracle_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                och_scalar value, int nthreads)
{
   const ptrdiff_t *st[1] = { strides }; void *pp[1] = { ptr };
   int es;
   if (dtype < 0 || dtype >= O_NTYPES) return -1;
   es = o_type_size[dtype];
   O_ELEMWISE_LOOP(1, ndims, size, st, pp, nthreads, { memcpy(q0, &value, es); })
   return 0;
}

static int o_is_fillnan(int dtype, const void *q)
{  /* real: isnan(x); complex: isnan(real) || isinf(imag) -- as in unary_ops.h:669-672 */
   switch (dtype)
   {  case O_HALF:    return isnan(o_half_to_float(*(const o_half *)q));
      case O_FLOAT:   return isnan(*(const float *)q);
      case O_DOUBLE:  return isnan(*(const double *)q);
      case O_CHALF:   return isnan(o_half_to_float(((const o_chalf *)q)->real)) || isinf(o_half_to_float(((const o_chalf *)q)->imag));
      case O_CFLOAT:  return isnan(((const o_cfloat *)q)->real) || isinf(((const o_cfloat *)q)->imag);
      case O_CDOUBLE: return isnan(((const o_cdouble *)q)->real) || isinf(((const o_cdouble *)q)->imag);
   }
   return 0;
}

int oracle_fill_nan(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                och_scalar value, int nthreads)
{
   const ptrdiff_t *st[1] = { strides }; void *pp[1] = { ptr };
   int es;
   if (dtype < O_HALF || dtype >= O_NTYPES) return -1;
   es = o_type_size[dtype];
   O_ELEMWISE_LOOP(1, ndims, size, st, pp, nthreads, { if (o_is_fillnan(dtype, q0)) memcpy(q0, &value, es); })
   return 0;
}

int oracle_masked_fill(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides1, void *ptr1,
                const ptrdiff_t *strides2, void *ptr2, och_scalar value, int nthreads)
{
   const ptrdiff_t *st[2] = { strides1, strides2 }; void *pp[2] = { ptr1, ptr2 };
   int es;
   if (dtype < 0 || dtype >= O_NTYPES) return -1;
   es = o_type_size[dtype];
   O_ELEMWISE_LOOP(2, ndims, size, st, pp, nthreads, { if (*(const o_bool *)q1) memcpy(q0, &value, es); })
   return 0;
}

/* ---- steps (template_steps.c:31-100): value = offset + index * step, evaluated in the
   parameter's arithmetic (int64 offset/step combine with the size_t index as unsigned
   64-bit), converted to the work type, then to the element type --------------------- */
static void o_store_from_uint64(int dtype, void *q, uint64_t v)
{
   switch (dtype)
   {  case O_BOOL:   *(o_bool *)q = (o_bool)v; break;     /* work type of bool is its 8-bit storage */
      case O_UINT8:  *(uint8_t *)q = (uint8_t)v; break;   case O_UINT16: *(uint16_t *)q = (uint16_t)v; break;
      case O_UINT32: *(uint32_t *)q = (uint32_t)v; break; case O_UINT64: *(uint64_t *)q = (uint64_t)v; break;
      case O_INT8:   *(int8_t *)q = (int8_t)v; break;     case O_INT16:  *(int16_t *)q = (int16_t)v; break;
      case O_INT32:  *(int32_t *)q = (int32_t)v; break;   case O_INT64:  *(int64_t *)q = (int64_t)v; break;
      case O_HALF:   *(o_half *)q = o_float_to_half((float)v); break;
      case O_FLOAT:  *(float *)q = (float)v; break;       case O_DOUBLE: *(double *)q = (double)v; break;
      case O_CHALF:  ((o_chalf *)q)->real = o_float_to_half((float)v); ((o_chalf *)q)->imag = o_float_to_half(0); break;
      case O_CFLOAT: ((o_cfloat *)q)->real = (float)v; ((o_cfloat *)q)->imag = 0; break;
      case O_CDOUBLE:((o_cdouble *)q)->real = (double)v; ((o_cdouble *)q)->imag = 0; break;
   }
}
static void o_store_part_from_double(int dtype, void *q, double v, int imag_part)
{
   switch (dtype)
   {  case O_BOOL:   *(o_bool *)q = (o_bool)v; break;
      case O_UINT8:  *(uint8_t *)q = (uint8_t)v; break;   case O_UINT16: *(uint16_t *)q = (uint16_t)v; break;
      case O_UINT32: *(uint32_t *)q = (uint32_t)v; break; case O_UINT64: *(uint64_t *)q = (uint64_t)v; break;
      case O_INT8:   *(int8_t *)q = (int8_t)v; break;     case O_INT16:  *(int16_t *)q = (int16_t)v; break;
      case O_INT32:  *(int32_t *)q = (int32_t)v; break;   case O_INT64:  *(int64_t *)q = (int64_t)v; break;
      case O_HALF:   *(o_half *)q = o_float_to_half((float)v); break;
      case O_FLOAT:  *(float *)q = (float)v; break;       case O_DOUBLE: *(double *)q = v; break;
      case O_CHALF:  if (imag_part) ((o_chalf *)q)->imag = o_float_to_half((float)v); else ((o_chalf *)q)->real = o_float_to_half((float)v); break;
      case O_CFLOAT: if (imag_part) ((o_cfloat *)q)->imag = (float)v; else ((o_cfloat *)q)->real = (float)v; break;
      case O_CDOUBLE:if (imag_part) ((o_cdouble *)q)->imag = v; else ((o_cdouble *)q)->real = v; break;
   }
}

#define O_STEPS_LOOP(...)                                                                     \
   {  size_t nelem = o_nelem(ndims, size);                                                    \
      if (nthreads < 1) nthreads = 1;                                                         \
      if ((size_t)nthreads > nelem) nthreads = (int)(nelem ? nelem : 1);                      \
      _Pragma("omp parallel num_threads(nthreads)")                                           \
      {  size_t a, b, index; o_iter it; int rank = 0, nt = 1;                                 \
         const ptrdiff_t *sa[1] = { strides }; void *pa[1] = { ptr };                         \
         O_OMP_RANK(rank, nt)                                                                 \
         o_thread_range(nelem, rank, nt, &a, &b);                                             \
         if (a < b)                                                                           \
         {  o_iter_init(&it, 1, ndims, size, sa, pa, a);                                      \
            for (index = a; index < b; index++) { char *q = it.p[0]; __VA_ARGS__ o_iter_carry(&it, 1); } \
         }                                                                                    \
      }                                                                                       \
   }
#ifdef _OPENMP
#define O_OMP_RANK(r, n) r = omp_get_thread_num(); n = omp_get_num_threads();
#else
#define O_OMP_RANK(r, n)
#endif

int oracle_steps_int64(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                int64_t offset, int64_t step, int nthreads)
{
   if (dtype < 0 || dtype >= O_NTYPES) return -1;
   O_STEPS_LOOP({ o_store_from_uint64(dtype, q, (uint64_t)offset + (uint64_t)index * (uint64_t)step); })
   return 0;
}

int oracle_steps_double(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                double offset, double step, int nthreads)
{
   if (dtype < 0 || dtype >= O_NTYPES) return -1;
   O_STEPS_LOOP({ o_store_part_from_double(dtype, q, offset + index * step, 0);
                  if (dtype >= O_CHALF) o_store_part_from_double(dtype, q, 0, 1); })
   return 0;
}

int oracle_steps_cdouble(int dtype, int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr,
                och_cdouble offset, och_cdouble step, int nthreads)
{
   if (dtype < 0 || dtype >= O_NTYPES) return -1;
   O_STEPS_LOOP({ o_store_part_from_double(dtype, q, offset.real + index * step.real, 0);
                  if (dtype >= O_CHALF) o_store_part_from_double(dtype, q, offset.imag + index * step.imag, 1); })
   return 0;
}
