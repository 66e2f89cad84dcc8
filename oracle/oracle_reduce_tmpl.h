/* TEST INFRASTRUCTURE (see oracle_types.h).
 * Per-type template of the reduction operations, included once per element type by
 * oracle_reduce.c (same parameter macros as oracle_ops_tmpl.h). For every operation it
 * defines three functions used by both the full and the axis reduction drivers:
 *    accumulate over a range of the traversal  (reduce_ops.h: init + accumulate code)
 *    combine two partial results                (reduce code)
 *    finalize and store in the result type      (finalize code + SOLID_ASSIGN)
 * restating solid/include/solid/core/generic/reduce_ops.h:139-1287; accumulation happens in
 * the work type of the RESULT type, exactly as the CPU templates do
 * (solid/include/solid/core/cpu/reduce_all.h:114-169).
 * Pinned by tests/test_oracle_ref.py against the reference macros (serial fold).
 */
#define RCAT_(a, b) a##b
#define RCAT(a, b) RCAT_(a, b)
#define RCAT3_(a, b, c) a##b##c
#define RCAT3(a, b, c) RCAT3_(a, b, c)
#define PT RCAT(o_t_, PN)
#define TOW(v)   RCAT3(o_cvt_, PN, RCAT(_, WN))(v)
#define FROMW(v) RCAT3(o_cvt_, WN, RCAT(_, PN))(v)
#define RNAME(op, part) RCAT3(o_red_, op, RCAT3(_, TN, part))

/* ACC: accumulator C type; RES: result C type; x: current element (const T);
   INIT may use x (first element of the range); STORE converts acc into *(RES *)result */
#define STRIP(...) __VA_ARGS__
#define RED(OP, ACC, RES, INIT, ACCUM, COMBINE, FINAL, STORE)                                \
   static void RNAME(OP, _acc)(int ndims, const size_t *size, const ptrdiff_t *strides, void *ptr, \
                               size_t start, size_t stop, const o_red_param *prm, void *out)  \
   {  ACC acc; const ptrdiff_t *st[1] = { strides }; void *pp[1] = { ptr }; int first = 1;    \
      memset(&acc, 0, sizeof(acc));                                                           \
      if (start >= stop) { T x; memset(&x, 0, sizeof(x)); (void)x; { STRIP INIT } } \
      O_RANGE_LOOP(1, ndims, size, st, pp, start, stop,                                       \
      {  const T x = *(const T *)q0;                                                          \
         if (first) { first = 0; { STRIP INIT } }                                                   \
         { STRIP ACCUM }                                                                            \
      })                                                                                      \
      (void)prm; *(ACC *)out = acc;                                                           \
   }                                                                                          \
   static void RNAME(OP, _cmb)(void *vres, const void *vpart)                                 \
   {  ACC *res = (ACC *)vres; const ACC *part = (const ACC *)vpart; { STRIP COMBINE } }             \
   static void RNAME(OP, _fin)(void *vacc, const o_red_param *prm, void *result)              \
   {  ACC acc = *(ACC *)vacc; { STRIP FINAL } { STRIP STORE } (void)prm; }                                \
   static const o_red_desc RNAME(OP, _desc) = { sizeof(ACC), RNAME(OP, _acc), RNAME(OP, _cmb), RNAME(OP, _fin) };

#if K_COMPLEX
typedef struct { W real, imag; } RCAT(o_cw_, TN);
#define CW RCAT(o_cw_, TN)
#define XR TOW(x.real)
#define XI TOW(x.imag)
#define NONZERO ((!(XR == 0)) || (!(XI == 0)))
#else
#if K_FLOAT
#define XV TOW(x)
#else
#define XV (x)
#endif
#define NONZERO (!(XV == 0))
#endif

/* ---------------- logical reductions: result bool ---------------- */
RED(any, o_bool, o_bool, (acc = 0;), (if (NONZERO) acc = 1;), (*res |= *part;), (), (*(o_bool *)result = acc;))
RED(all, o_bool, o_bool, (acc = 1;), (if (!NONZERO) acc = 0;), (*res &= *part;), (), (*(o_bool *)result = acc;))
RED(nnz, uint64_t, uint64_t, (acc = 0;), (if (NONZERO) acc++;), (*res += *part;), (), (*(uint64_t *)result = acc;))

#if K_FLOAT
RED(all_finite, o_bool, o_bool, (acc = 1;), (if (!isfinite(XV)) acc = 0;), (*res &= *part;), (), (*(o_bool *)result = acc;))
RED(any_inf, o_bool, o_bool, (acc = 0;), (if (isinf(XV)) acc = 1;), (*res |= *part;), (), (*(o_bool *)result = acc;))
RED(any_nan, o_bool, o_bool, (acc = 0;), (if (isnan(XV)) acc = 1;), (*res |= *part;), (), (*(o_bool *)result = acc;))
RED(nnz_nan, uint64_t, uint64_t, (acc = 0;), ({ W t = XV; if ((!isnan(t)) && (t != 0)) acc++; }), (*res += *part;), (), (*(uint64_t *)result = acc;))
#elif K_COMPLEX
RED(all_finite, o_bool, o_bool, (acc = 1;), (if ((!isfinite(XR)) || (!isfinite(XI))) acc = 0;), (*res &= *part;), (), (*(o_bool *)result = acc;))
RED(any_inf, o_bool, o_bool, (acc = 0;), (if (isinf(XR) || isinf(XI)) acc = 1;), (*res |= *part;), (), (*(o_bool *)result = acc;))
RED(any_nan, o_bool, o_bool, (acc = 0;), (if (isnan(XR) || isnan(XI)) acc = 1;), (*res |= *part;), (), (*(o_bool *)result = acc;))
RED(nnz_nan, uint64_t, uint64_t, (acc = 0;), ({ W a = XR, b = XI; /* the parts are passed through the part-type conversion once more (reduce_ops.h:329-330); for chalf this truncates them to an integer bit pattern first */ if ((!isnan(a)) && (!isnan(b)) && ((TOW((PT)a) != 0) || (TOW((PT)b) != 0))) acc++; }), (*res += *part;), (), (*(uint64_t *)result = acc;))
#endif

/* bounds are given in the tensor's type and compared in the work type */
#if K_COMPLEX
#define LO_R TOW(((const T *)&prm->b1)->real)
#define LO_I TOW(((const T *)&prm->b1)->imag)
#define HI_R TOW(((const T *)&prm->b2)->real)
#define HI_I TOW(((const T *)&prm->b2)->imag)
#define RANGE(OP, FAIL) RED(OP, o_bool, o_bool, (acc = 1;), ({ W re = XR, im = XI; (void)im; if (FAIL) acc = 0; }), (*res &= *part;), (), (*(o_bool *)result = acc;))
RANGE(all_lt, ((re > LO_R) || ((re == LO_R) && (im >= LO_I))))
RANGE(all_le, ((re > LO_R) || ((re == LO_R) && (im >  LO_I))))
RANGE(all_gt, ((re < LO_R) || ((re == LO_R) && (im <= LO_I))))
RANGE(all_ge, ((re < LO_R) || ((re == LO_R) && (im <  LO_I))))
RANGE(all_gtlt, ((re < LO_R) || (re > HI_R) || ((re == LO_R) && (im <= LO_I)) || ((re == HI_R) && (im >= HI_I))))
RANGE(all_gtle, ((re < LO_R) || (re > HI_R) || ((re == LO_R) && (im <= LO_I)) || ((re == HI_R) && (im >  HI_I))))
RANGE(all_gelt, ((re < LO_R) || (re > HI_R) || ((re == LO_R) && (im <  LO_I)) || ((re == HI_R) && (im >= HI_I))))
RANGE(all_gele, ((re < LO_R) || (re > HI_R) || ((re == LO_R) && (im <  LO_I)) || ((re == HI_R) && (im >  HI_I))))
#undef LO_R
#undef LO_I
#undef HI_R
#undef HI_I
#else
#if K_FLOAT
#define LO TOW(*(const T *)&prm->b1)
#define HI TOW(*(const T *)&prm->b2)
#else
#define LO (*(const T *)&prm->b1)
#define HI (*(const T *)&prm->b2)
#endif
#define RANGE(OP, FAIL) RED(OP, o_bool, o_bool, (acc = 1;), (if (FAIL) acc = 0;), (*res &= *part;), (), (*(o_bool *)result = acc;))
RANGE(all_lt, (XV >= LO))
RANGE(all_le, (XV >  LO))
RANGE(all_gt, (XV <= LO))
RANGE(all_ge, (XV <  LO))
RANGE(all_gtlt, ((XV <= LO) || (XV >= HI)))
RANGE(all_gtle, ((XV <= LO) || (XV >  HI)))
RANGE(all_gelt, ((XV <  LO) || (XV >= HI)))
RANGE(all_gele, ((XV <  LO) || (XV >  HI)))
#undef LO
#undef HI
#endif
#undef RANGE

/* ---------------- sums and products ---------------- */
#if K_BOOL || K_UINT
RED(sum, uint64_t, uint64_t, (acc = 0;), (acc += XV;), (*res += *part;), (), (*(uint64_t *)result = acc;))
RED(prod, uint64_t, uint64_t, (acc = 1;), (acc *= XV;), (*res *= *part;), (), (*(uint64_t *)result = acc;))
RED(sum_abs, uint64_t, uint64_t, (acc = 0;), (acc += XV;), (*res += *part;), (), (*(uint64_t *)result = acc;))
#elif K_SINT
RED(sum, int64_t, int64_t, (acc = 0;), (acc = (int64_t)((uint64_t)acc + (uint64_t)(int64_t)x);), (*res = (int64_t)((uint64_t)*res + (uint64_t)*part);), (), (*(int64_t *)result = acc;))
RED(prod, int64_t, int64_t, (acc = 1;), (acc = (int64_t)((uint64_t)acc * (uint64_t)(int64_t)x);), (*res = (int64_t)((uint64_t)*res * (uint64_t)*part);), (), (*(int64_t *)result = acc;))
RED(sum_abs, uint64_t, uint64_t, (acc = 0;), ({ if (x < 0) acc -= x; else acc += x; }), (*res += *part;), (), (*(uint64_t *)result = acc;))
#elif K_FLOAT
RED(sum, W, T, (acc = 0;), (acc += XV;), (*res += *part;), (), (*(T *)result = FROMW(acc);))
RED(prod, W, T, (acc = 1;), (acc *= XV;), (*res *= *part;), (), (*(T *)result = FROMW(acc);))
RED(sum_nan, W, T, (acc = 0;), ({ W t = XV; if (!isnan(t)) acc += t; }), (*res += *part;), (), (*(T *)result = FROMW(acc);))
RED(prod_nan, W, T, (acc = 1;), ({ W t = XV; if (!isnan(t)) acc *= t; }), (*res *= *part;), (), (*(T *)result = FROMW(acc);))
RED(sum_abs, W, T, (acc = 0;), (acc += MF(fabs)(XV);), (*res += *part;), (), (*(T *)result = FROMW(acc);))
RED(sum_abs_nan, W, T, (acc = 0;), ({ W t = XV; if (!isnan(t)) acc += MF(fabs)(t); }), (*res += *part;), (), (*(T *)result = FROMW(acc);))
#else
#define CSTORE { ((T *)result)->real = FROMW(acc.real); ((T *)result)->imag = FROMW(acc.imag); }
RED(sum, CW, T, ({ acc.real = 0; acc.imag = 0; }), ({ acc.real += XR; acc.imag += XI; }), ({ res->real += part->real; res->imag += part->imag; }), (), (CSTORE))
RED(prod, CW, T, ({ acc.real = 1; acc.imag = 0; }), ({ W a = XR, b = XI, t = acc.real; acc.real = t * a - acc.imag * b; acc.imag = t * b + acc.imag * a; }), ({ W t = res->real; res->real = t * part->real - res->imag * part->imag; res->imag = t * part->imag + res->imag * part->real; }), (), (CSTORE))
RED(sum_nan, CW, T, ({ acc.real = 0; acc.imag = 0; }), ({ W a = XR, b = XI; if ((!isnan(a)) && (!isnan(b))) { acc.real += a; acc.imag += b; } }), ({ res->real += part->real; res->imag += part->imag; }), (), (CSTORE))
/* literal restatement, including the minus sign in the imaginary update (reduce_ops.h:784) */
RED(prod_nan, CW, T, ({ acc.real = 1; acc.imag = 0; }), ({ W a = XR, b = XI, t; if ((!isnan(a)) && (!isnan(b))) { t = acc.real; acc.real = t * a - acc.imag * b; acc.imag = t * b - acc.imag * a; } }), ({ W t = res->real; res->real = t * part->real - res->imag * part->imag; res->imag = t * part->imag + res->imag * part->real; }), (), (CSTORE))
RED(sum_abs, W, PT, (acc = 0;), (acc += MF(hypot)(XR, XI);), (*res += *part;), (), (*(PT *)result = FROMW(acc);))
RED(sum_abs_nan, W, PT, (acc = 0;), ({ W a = XR, b = XI; if ((!isnan(a)) && (!isnan(b))) acc += MF(hypot)(a, b); }), (*res += *part;), (), (*(PT *)result = FROMW(acc);))
#endif

/* ---------------- extrema: the accumulator starts from the first element ---------------- */
#if K_BOOL || K_UINT || K_SINT
RED(maximum, T, T, (acc = x;), (if (acc < x) acc = x;), (if (*res < *part) *res = *part;), (), (*(T *)result = acc;))
RED(minimum, T, T, (acc = x;), (if (acc > x) acc = x;), (if (*res > *part) *res = *part;), (), (*(T *)result = acc;))
#if K_SINT
#define ABSV ((UT)((x < 0) ? -(x) : (x)))
RED(maximum_abs, UT, UT, (acc = ABSV;), ({ UT a = ABSV; if (acc < a) acc = a; }), (if (*res < *part) *res = *part;), (), (*(UT *)result = acc;))
RED(minimum_abs, UT, UT, (acc = ABSV;), ({ UT a = ABSV; if (acc > a) acc = a; }), (if (*res > *part) *res = *part;), (), (*(UT *)result = acc;))
#undef ABSV
#else
RED(maximum_abs, T, T, (acc = x;), (if (acc < x) acc = x;), (if (*res < *part) *res = *part;), (), (*(T *)result = acc;))
RED(minimum_abs, T, T, (acc = x;), (if (acc > x) acc = x;), (if (*res > *part) *res = *part;), (), (*(T *)result = acc;))
#endif
#elif K_FLOAT
RED(maximum, W, T, (acc = XV;), ({ W t = XV; if ((!isnan(t)) && (!(acc >= t))) acc = t; }), ({ W t = *part; if ((!isnan(t)) && (!(*res >= t))) *res = t; }), (), (*(T *)result = FROMW(acc);))
RED(minimum, W, T, (acc = XV;), ({ W t = XV; if ((!isnan(t)) && (!(acc <= t))) acc = t; }), ({ W t = *part; if ((!isnan(t)) && (!(*res <= t))) *res = t; }), (), (*(T *)result = FROMW(acc);))
RED(maximum_abs, W, T, (acc = MF(fabs)(XV);), ({ W t = MF(fabs)(XV); if ((!isnan(t)) && (!(acc >= t))) acc = t; }), ({ W t = *part; if ((!isnan(t)) && (!(*res >= t))) *res = t; }), (), (*(T *)result = FROMW(acc);))
RED(minimum_abs, W, T, (acc = MF(fabs)(XV);), ({ W t = MF(fabs)(XV); if ((!isnan(t)) && (!(acc <= t))) acc = t; }), ({ W t = *part; if ((!isnan(t)) && (!(*res <= t))) *res = t; }), (), (*(T *)result = FROMW(acc);))
#else
RED(maximum, CW, T, ({ acc.real = XR; acc.imag = XI; }), ({ W a = XR, b = XI;
      if ((!isnan(a)) && (!isnan(b)) && ((!(acc.real >= a)) || ((!(acc.real < a)) && (!(acc.real > a)) && (!(acc.imag >= b))) || (isnan(acc.imag))))
      { acc.real = a; acc.imag = b; } }), ({ W a = part->real, b = part->imag, r = res->real;
      if ((!isnan(a)) && (!isnan(b)) && ((!(r >= a)) || ((!(r < a)) && (!(r > a)) && (!(res->imag >= b))) || (isnan(res->imag))))
      { res->real = a; res->imag = b; } }), (), (CSTORE))
RED(minimum, CW, T, ({ acc.real = XR; acc.imag = XI; }), ({ W a = XR, b = XI;
      if ((!isnan(a)) && (!isnan(b)) && ((!(acc.real <= a)) || ((!(acc.real < a)) && (!(acc.real > a)) && (!(acc.imag <= b))) || (isnan(acc.imag))))
      { acc.real = a; acc.imag = b; } }), ({ W a = part->real, b = part->imag, r = res->real;
      if ((!isnan(a)) && (!isnan(b)) && ((!(r <= a)) || ((!(r < a)) && (!(r > a)) && (!(res->imag <= b))) || (isnan(res->imag))))
      { res->real = a; res->imag = b; } }), (), (CSTORE))
RED(maximum_abs, W, PT, (acc = MF(hypot)(XR, XI);), ({ W t = MF(hypot)(XR, XI); if ((!isnan(t)) && (!(acc >= t))) acc = t; }), ({ W t = *part; if ((!isnan(t)) && (!(*res >= t))) *res = t; }), (), (*(PT *)result = FROMW(acc);))
RED(minimum_abs, W, PT, (acc = MF(hypot)(XR, XI);), ({ W t = MF(hypot)(XR, XI); if ((!isnan(t)) && (!(acc <= t))) acc = t; }), ({ W t = *part; if ((!isnan(t)) && (!(*res <= t))) *res = t; }), (), (*(PT *)result = FROMW(acc);))
#endif

/* ---------------- norms ---------------- */
#if K_BOOL || K_UINT || K_SINT
/* pow of the CPU function table is powf, also for the double-typed integer norm */
RED(norm, double, double, (acc = 0;), ({ double t = (double)(XV); t *= t; acc += powf(t, prm->p / 2); }), (*res += *part;), (acc = powf(acc, 1 / prm->p);), (*(double *)result = acc;))
RED(norm2, double, double, (acc = 0;), ({ double t = (double)(XV); acc += t * t; }), (*res += *part;), (acc = sqrt(acc);), (*(double *)result = acc;))
#elif K_FLOAT
/* pow of the CPU function table is powf for every type */
RED(norm, W, T, (acc = 0;), ({ W t = XV; t *= t; acc += powf(t, (W)(prm->p / 2)); }), (*res += *part;), (acc = powf(acc, (W)(1 / prm->p));), (*(T *)result = FROMW(acc);))
RED(norm_nan, W, T, (acc = 0;), ({ W t = XV; if (!isnan(t)) { t *= t; acc += powf(t, (W)(prm->p / 2)); } }), (*res += *part;), (acc = powf(acc, (W)(1 / prm->p));), (*(T *)result = FROMW(acc);))
RED(norm2, W, T, (acc = 0;), ({ W t = XV; acc += t * t; }), (*res += *part;), (acc = MF(sqrt)(acc);), (*(T *)result = FROMW(acc);))
RED(norm2_nan, W, T, (acc = 0;), ({ W t = XV; if (!isnan(t)) acc += t * t; }), (*res += *part;), (acc = MF(sqrt)(acc);), (*(T *)result = FROMW(acc);))
#else
RED(norm, W, PT, (acc = 0;), ({ W a = XR, b = XI, t = (a * a) + (b * b); acc += powf(t, (W)(prm->p / 2)); }), (*res += *part;), (acc = powf(acc, (W)(1 / prm->p));), (*(PT *)result = FROMW(acc);))
RED(norm_nan, W, PT, (acc = 0;), ({ W a = XR, b = XI, t = (a * a) + (b * b); if (!isnan(t)) acc += powf(t, (W)(prm->p / 2)); }), (*res += *part;), (acc = powf(acc, (W)(1 / prm->p));), (*(PT *)result = FROMW(acc);))
RED(norm2, W, PT, (acc = 0;), ({ W a = XR, b = XI; acc += (a * a) + (b * b); }), (*res += *part;), (acc = MF(sqrt)(acc);), (*(PT *)result = FROMW(acc);))
RED(norm2_nan, W, PT, (acc = 0;), ({ W a = XR, b = XI, t; t = (a * a) + (b * b); if (!isnan(t)) acc += t; }), (*res += *part;), (acc = MF(sqrt)(acc);), (*(PT *)result = FROMW(acc);))
#endif

#undef RED
#undef STRIP
#undef NONZERO
#ifdef XV
#undef XV
#endif
#ifdef XR
#undef XR
#undef XI
#undef CW
#undef CSTORE
#endif
#undef PT
#undef TOW
#undef FROMW
#undef RNAME
#undef RCAT
#undef RCAT_
#undef RCAT3
#undef RCAT3_
