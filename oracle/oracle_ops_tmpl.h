/* TEST INFRASTRUCTURE (see oracle_types.h).
 * Per-type template: included once per element type by oracle_elemwise.c with
 *   TN  type name token          T   C type            UT  unsigned twin (integers)
 *   K_BOOL / K_UINT / K_SINT / K_FLOAT / K_COMPLEX     exactly one is 1
 *   W   work type of a real value or of a complex part (float for half)
 *   PN  name token of the real part type (complex) or TN (real)
 *   MF(f) math function in W precision
 * Restates, operation by operation,
 *   solid/include/solid/core/generic/binary_ops.h:112-520,
 *   solid/include/solid/core/generic/unary_ops.h:203-672,
 *   function tables solid/include/solid/core/cpu/unary_ops_cpu.h:24-140,
 *   type tables solid/src/core/cpu/template_binary.c:37-260 and template_unary.c:35-260.
 * Pinned by tests/test_oracle_ref.py against the reference macros themselves.
 */

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define CAT3_(a, b, c) a##b##c
#define CAT3(a, b, c) CAT3_(a, b, c)
#define PT CAT(o_t_, PN)                               /* part C type */
#define TOW(v)   CAT3(o_cvt_, PN, CAT(_, WN))(v)       /* part -> work type */
#define FROMW(v) CAT3(o_cvt_, WN, CAT(_, PN))(v)       /* work type -> part */

/* ---------------- loop shells ---------------- */
#define BIN_LOOP(NAME, TB, TR, ...)                                                           \
   static int CAT3(o_bin_, NAME, CAT(_, TN))(int ndims, const size_t *size,                  \
         const ptrdiff_t *s1, void *p1, const ptrdiff_t *s2, void *p2, const ptrdiff_t *s3, void *p3) \
   {  const ptrdiff_t *st[3] = { s1, s2, s3 }; void *pp[3] = { p1, p2, p3 };                 \
      O_ELEMWISE_LOOP(3, ndims, size, st, pp, 0,                                             \
      {  const T x = *(const T *)q0; const TB y = *(const TB *)q1; TR z; __VA_ARGS__ *(TR *)q2 = z; }) \
      return 0;                                                                              \
   }
#define UN_LOOP(NAME, TR, ...)                                                               \
   static int CAT3(o_un_, NAME, CAT(_, TN))(int ndims, const size_t *size,                   \
         const ptrdiff_t *s1, void *p1, const ptrdiff_t *s2, void *p2, int nthreads)         \
   {  const ptrdiff_t *st[2] = { s1, s2 }; void *pp[2] = { p1, p2 };                         \
      O_ELEMWISE_LOOP(2, ndims, size, st, pp, nthreads,                                      \
      {  const T x = *(const T *)q0; TR y; __VA_ARGS__ *(TR *)q1 = y; })                            \
      return 0;                                                                              \
   }

/* =====================================================================
 * BOOL
 * ===================================================================== */
#if K_BOOL
BIN_LOOP(add, T, T, z = x | y;)
BIN_LOOP(subtract, T, T, z = x & (T)~y;)
BIN_LOOP(multiply, T, T, z = x & y;)
BIN_LOOP(true_divide, T, T, z = x & y;)
BIN_LOOP(mod, T, T, z = 0; (void)x; (void)y;)
BIN_LOOP(power, int16_t, T, z = (T)((x != 0) | (y == 0));)
BIN_LOOP(bitwise_and, T, T, z = x & y;)
BIN_LOOP(bitwise_or, T, T, z = x | y;)
BIN_LOOP(bitwise_xor, T, T, z = x ^ y;)
BIN_LOOP(bitshift_left, int8_t, T, z = (y == 0) ? (x & 1) : 0;)
BIN_LOOP(bitshift_right, int8_t, T, z = (y == 0) ? (x & 1) : 0;)
BIN_LOOP(lt, T, o_bool, z = (x <  y) ? 1 : 0;)
BIN_LOOP(le, T, o_bool, z = (x <= y) ? 1 : 0;)
BIN_LOOP(eq, T, o_bool, z = (x == y) ? 1 : 0;)
BIN_LOOP(ne, T, o_bool, z = (x != y) ? 1 : 0;)
BIN_LOOP(ge, T, o_bool, z = (x >= y) ? 1 : 0;)
BIN_LOOP(gt, T, o_bool, z = (x >  y) ? 1 : 0;)
UN_LOOP(logical_not, T, y = x ^ 1;)
UN_LOOP(fabs, T, y = x;)
UN_LOOP(sign, T, y = x;)
UN_LOOP(isinf, o_bool, y = 0; (void)x;)
UN_LOOP(isnan, o_bool, y = 0; (void)x;)
UN_LOOP(isfinite, o_bool, y = 1; (void)x;)
UN_LOOP(isposinf, o_bool, y = 0; (void)x;)
UN_LOOP(isneginf, o_bool, y = 0; (void)x;)
#endif

/* =====================================================================
 * INTEGERS
 * ===================================================================== */
#if K_UINT || K_SINT
/* wrap-around arithmetic is done on the unsigned twin */
BIN_LOOP(add, T, T, z = (T)((UT)x + (UT)y);)
BIN_LOOP(subtract, T, T, z = (T)((UT)x - (UT)y);)
BIN_LOOP(multiply, T, T, z = (T)((UT)((UT)x * (UT)y));)
BIN_LOOP(true_divide, T, T, z = (y == 0) ? 0 : (T)(x / y);)
BIN_LOOP(bitwise_and, T, T, z = x & y;)
BIN_LOOP(bitwise_or, T, T, z = x | y;)
BIN_LOOP(bitwise_xor, T, T, z = x ^ y;)
BIN_LOOP(bitshift_left, int8_t, T, z = (y < 0) ? (T)(x >> -y) : (T)(x << y);)
BIN_LOOP(bitshift_right, int8_t, T, z = (y < 0) ? (T)(x << -y) : (T)(x >> y);)
BIN_LOOP(lt, T, o_bool, z = (x <  y) ? 1 : 0;)
BIN_LOOP(le, T, o_bool, z = (x <= y) ? 1 : 0;)
BIN_LOOP(eq, T, o_bool, z = (x == y) ? 1 : 0;)
BIN_LOOP(ne, T, o_bool, z = (x != y) ? 1 : 0;)
BIN_LOOP(ge, T, o_bool, z = (x >= y) ? 1 : 0;)
BIN_LOOP(gt, T, o_bool, z = (x >  y) ? 1 : 0;)
BIN_LOOP(min, T, T, z = (x <= y) ? x : y;)
BIN_LOOP(max, T, T, z = (x >= y) ? x : y;)
BIN_LOOP(power, int16_t, T,
   {  T b = x; int64_t e = y; z = (T)(e >= 0);
      while (e > 0) { if (e & 1) z = (T)((UT)z * (UT)b); e >>= 1; b = (T)((UT)b * (UT)b); }
   })
#if K_UINT
BIN_LOOP(mod, T, T, z = (y == 0) ? 0 : (T)(x % y);)
#else
/* the sign test of x*y is made on the product in the promoted type (int for 8/16 bit) */
#define NEGPROD(a, b) ((sizeof(T) < 4) ? (((int)(a) * (int)(b)) < 0) : ((T)((UT)(a) * (UT)(b)) < 0))
BIN_LOOP(divide, T, T,
   {  if (y == 0) z = 0;
      else if (sizeof(T) < 4) { int a = x, b = y; z = (T)((a - (a * b < 0) * (b + ((b < 0) - (b > 0)))) / b); }
      else { T a = (T)((UT)x - (UT)(NEGPROD(x, y) * (T)(y + ((y < 0) - (y > 0))))); z = (T)(a / y); }
   })
BIN_LOOP(floor_divide, T, T,
   {  if (y == 0) z = 0;
      else { T a = x; a = (T)((UT)a - (UT)(NEGPROD(a, y) * (T)(y + ((y < 0) - (y > 0))))); z = (T)(a / y); }
   })
BIN_LOOP(fmod, T, T, z = (y == 0) ? 0 : (T)(x % y);)
BIN_LOOP(mod, T, T,
   {  if (y == 0) z = 0;
      else { T r = (T)(x % y); z = (T)((UT)r + (UT)((NEGPROD(x, y) && (r != 0)) * y)); }
   })
#undef NEGPROD
#endif

/* unary */
UN_LOOP(bitwise_not, T, y = (T)~x;)
#if K_SINT
UN_LOOP(negative, T, y = (T)((UT)0 - (UT)x);)
UN_LOOP(fabs, T, y = (T)((UT)((x >= 0) - (x < 0)) * (UT)x);)
UN_LOOP(sign, T, y = (T)((x > 0) - (x < 0));)
UN_LOOP(sqrt,  T, y = (x <= 0) ? 0 : (T)sqrt((double)x);)
UN_LOOP(log,   T, y = (x <= 0) ? 0 : (T)log((double)x);)
UN_LOOP(log2,  T, y = (x <= 0) ? 0 : (T)log2((double)x);)
UN_LOOP(log10, T, y = (x <= 0) ? 0 : (T)log10((double)x);)
UN_LOOP(log1p, T, { double d = x; y = (d <= -1) ? 0 : (T)log1p(d); })
#else
UN_LOOP(fabs, T, y = x;)
UN_LOOP(sign, T, y = (T)(x > 0);)
UN_LOOP(sqrt,  T, y = (T)sqrt((double)x);)
UN_LOOP(log,   T, y = (T)log((double)x);)
UN_LOOP(log2,  T, y = (T)log2((double)x);)
UN_LOOP(log10, T, y = (T)log10((double)x);)
UN_LOOP(log1p, T, y = (T)log1p((double)x);)
#endif
UN_LOOP(reciprocal, T, y = (x == 0) ? 0 : (T)(1 / x);)
UN_LOOP(square, T, y = (T)((UT)x * (UT)x);)
#define INT_VIA_DOUBLE(NAME, FN) UN_LOOP(NAME, T, y = (T)FN((double)x);)
INT_VIA_DOUBLE(sin, sin)       INT_VIA_DOUBLE(cos, cos)       INT_VIA_DOUBLE(tan, tan)
INT_VIA_DOUBLE(sinh, sinh)     INT_VIA_DOUBLE(cosh, cosh)     INT_VIA_DOUBLE(tanh, tanh)
INT_VIA_DOUBLE(arcsin, asin)   INT_VIA_DOUBLE(arccos, acos)   INT_VIA_DOUBLE(arctan, atan)
INT_VIA_DOUBLE(arcsinh, asinh) INT_VIA_DOUBLE(arccosh, acosh) INT_VIA_DOUBLE(arctanh, atanh)
INT_VIA_DOUBLE(cbrt, cbrt)     INT_VIA_DOUBLE(exp, exp)       INT_VIA_DOUBLE(exp2, exp2)
INT_VIA_DOUBLE(expm1, expm1)
UN_LOOP(exp10, T, y = (T)exp(2.3025850929940459 * (double)x);)
#undef INT_VIA_DOUBLE
UN_LOOP(isinf, o_bool, y = 0; (void)x;)
UN_LOOP(isnan, o_bool, y = 0; (void)x;)
UN_LOOP(isfinite, o_bool, y = 1; (void)x;)
UN_LOOP(isposinf, o_bool, y = 0; (void)x;)
UN_LOOP(isneginf, o_bool, y = 0; (void)x;)
#endif

/* =====================================================================
 * REAL FLOATING POINT (half computes in float)
 * ===================================================================== */
#if K_FLOAT
BIN_LOOP(add, T, T, z = FROMW(TOW(x) + TOW(y));)
BIN_LOOP(subtract, T, T, z = FROMW(TOW(x) - TOW(y));)
BIN_LOOP(multiply, T, T, z = FROMW(TOW(x) * TOW(y));)
BIN_LOOP(true_divide, T, T, z = FROMW(TOW(x) / TOW(y));)
BIN_LOOP(floor_divide, T, T, { W a = TOW(x), b = TOW(y); z = FROMW(MF(floor)(a / b)); })
BIN_LOOP(mod, T, T, { W a = TOW(x), b = TOW(y), q; q = MF(floor)(a / b); z = FROMW((a - q * b)); })
BIN_LOOP(fmod, T, T, { W a = TOW(x), b = TOW(y); z = FROMW(fmod(a, b)); })
BIN_LOOP(power, T, T, { W a = TOW(x), b = TOW(y); z = FROMW(powf(a, b)); })
BIN_LOOP(lt, T, o_bool, z = (TOW(x) <  TOW(y)) ? 1 : 0;)
BIN_LOOP(le, T, o_bool, z = (TOW(x) <= TOW(y)) ? 1 : 0;)
BIN_LOOP(eq, T, o_bool, z = (TOW(x) == TOW(y)) ? 1 : 0;)
BIN_LOOP(ne, T, o_bool, z = (TOW(x) != TOW(y)) ? 1 : 0;)
BIN_LOOP(ge, T, o_bool, z = (TOW(x) >= TOW(y)) ? 1 : 0;)
BIN_LOOP(gt, T, o_bool, z = (TOW(x) >  TOW(y)) ? 1 : 0;)
BIN_LOOP(min,  T, T, { W a = TOW(x), b = TOW(y); if (isnan(b) || (b <  a)) a = b; z = FROMW(a); })
BIN_LOOP(max,  T, T, { W a = TOW(x), b = TOW(y); if (isnan(b) || (b >  a)) a = b; z = FROMW(a); })
BIN_LOOP(fmin, T, T, { W a = TOW(x), b = TOW(y); if (isnan(a) || (b <= a)) a = b; z = FROMW(a); })
BIN_LOOP(fmax, T, T, { W a = TOW(x), b = TOW(y); if (isnan(a) || (b >= a)) a = b; z = FROMW(a); })

UN_LOOP(negative, T, y = FROMW(-1 * TOW(x));)
UN_LOOP(reciprocal, T, y = FROMW(1. / TOW(x));)
UN_LOOP(square, T, { W a = TOW(x); y = FROMW(a * a); })
UN_LOOP(fabs, T, y = FROMW(MF(fabs)(TOW(x)));)
UN_LOOP(sign, T, { W a = TOW(x); if (isnan(a)) y = x; else y = FROMW((a > 0) - (a < 0)); })
#define REAL_FUN(NAME, FN) UN_LOOP(NAME, T, y = FROMW(MF(FN)(TOW(x)));)
REAL_FUN(sin, sin)       REAL_FUN(cos, cos)       REAL_FUN(tan, tan)
REAL_FUN(sinh, sinh)     REAL_FUN(cosh, cosh)     REAL_FUN(tanh, tanh)
REAL_FUN(arcsin, asin)   REAL_FUN(arccos, acos)   REAL_FUN(arctan, atan)
REAL_FUN(arcsinh, asinh) REAL_FUN(arccosh, acosh) REAL_FUN(arctanh, atanh)
REAL_FUN(sqrt, sqrt)     REAL_FUN(cbrt, cbrt)     REAL_FUN(exp, exp)      REAL_FUN(exp2, exp2)
REAL_FUN(expm1, expm1)   REAL_FUN(log, log)       REAL_FUN(log2, log2)    REAL_FUN(log10, log10)
REAL_FUN(log1p, log1p)   REAL_FUN(ceil, ceil)     REAL_FUN(floor, floor)  REAL_FUN(trunc, trunc)
REAL_FUN(round, round)
#undef REAL_FUN
UN_LOOP(exp10, T, y = FROMW(MF(exp)(((W)2.3025850929940459) * TOW(x)));)
UN_LOOP(isinf, o_bool, y = isinf(TOW(x)) ? 1 : 0;)
UN_LOOP(isnan, o_bool, y = isnan(TOW(x)) ? 1 : 0;)
UN_LOOP(isfinite, o_bool, y = isfinite(TOW(x)) ? 1 : 0;)
UN_LOOP(isposinf, o_bool, { W a = TOW(x); y = ((a > 0) && isinf(a)) ? 1 : 0; })
UN_LOOP(isneginf, o_bool, { W a = TOW(x); y = ((a < 0) && isinf(a)) ? 1 : 0; })
#endif

/* =====================================================================
 * COMPLEX (parts are converted to W, combined with separately rounded
 * operations, and converted back)
 * ===================================================================== */
#if K_COMPLEX
#define XR TOW(x.real)
#define XI TOW(x.imag)
#define YR TOW(y.real)
#define YI TOW(y.imag)
#define SETZ(re, im) { z.real = FROMW(re); z.imag = FROMW(im); }
#define SETY(re, im) { y.real = FROMW(re); y.imag = FROMW(im); }
BIN_LOOP(add, T, T, SETZ(XR + YR, XI + YI))
BIN_LOOP(subtract, T, T, SETZ(XR - YR, XI - YI))
BIN_LOOP(multiply, T, T, { W a = XR, b = XI, c = YR, d = YI; SETZ(a * c - b * d, a * d + c * b) })
BIN_LOOP(true_divide, T, T,
   {  W a = XR, b = XI, c = YR, d = YI, r = c * c + d * d; SETZ((a * c + b * d) / r, (b * c - a * d) / r) })
BIN_LOOP(power, T, T,
   {  W a = XR, b = XI, c = YR, d = YI, s = a * a + b * b, lr, li;
      if (s == 0) { z.real = FROMW((c == 0) && (d == 0)); z.imag = FROMW(0); }
      else
      {  li = MF(atan2)(b, a); lr = MF(log)(s) * 0.5;
         a = c * lr - d * li; b = c * li + d * lr;
         s = MF(exp)(a); a = s * MF(cos)(b); b = s * MF(sin)(b);
         SETZ(a, b)
      }
   })
BIN_LOOP(lt, T, o_bool, { W a = XR, c = YR; z = (a != c) ? (a < c) : (XI <  YI); })
BIN_LOOP(le, T, o_bool, { W a = XR, c = YR; z = (a != c) ? (a < c) : (XI <= YI); })
BIN_LOOP(ge, T, o_bool, { W a = XR, c = YR; z = (a != c) ? (a > c) : (XI >= YI); })
BIN_LOOP(gt, T, o_bool, { W a = XR, c = YR; z = (a != c) ? (a > c) : (XI >  YI); })
BIN_LOOP(eq, T, o_bool, z = ((XR == YR) && (XI == YI)) ? 1 : 0;)
BIN_LOOP(ne, T, o_bool, z = ((XR != YR) || (XI != YI)) ? 1 : 0;)
#define PICK(cond) { W a = XR, b = XI, c = YR, d = YI; if (cond) SETZ(c, d) else SETZ(a, b) }
BIN_LOOP(min,  T, T, PICK((isnan(c) || isnan(d)) || (c < a) || ((c == a) && (d < b))))
BIN_LOOP(max,  T, T, PICK((isnan(c) || isnan(d)) || (c > a) || ((c == a) && (d > b))))
BIN_LOOP(fmin, T, T, PICK(((c < a) || isnan(a)) || ((a == c) && ((d < b) || isnan(b)))))
BIN_LOOP(fmax, T, T, PICK(((c > a) || isnan(a)) || ((a == c) && ((d > b) || isnan(b)))))
#undef PICK

UN_LOOP(negative, T, SETY(-1 * XR, -1 * XI))
UN_LOOP(conj, T, { y.real = x.real; y.imag = FROMW(-1 * XI); })
UN_LOOP(reciprocal, T, { W a = XR, b = XI, s = 1. / ((a * a) + (b * b)); SETY(a * s, b * s * -1) })
UN_LOOP(sin,  T, { W a = XR, b = XI; SETY(MF(sin)(a) * MF(cosh)(b), MF(cos)(a) * MF(sinh)(b)) })
UN_LOOP(cos,  T, { W a = XR, b = XI; SETY(MF(cos)(a) * MF(cosh)(b), MF(sin)(a) * MF(sinh)(b) * -1) })
UN_LOOP(tan,  T, { W a = 2 * XR, b = 2 * XI, r; r = (MF(cos)(a) + MF(cosh)(b)); SETY(MF(sin)(a) / r, MF(sinh)(b) / r) })
UN_LOOP(sinh, T, { W a = XR, b = XI; SETY(MF(sinh)(a) * MF(cos)(b), MF(cosh)(a) * MF(sin)(b)) })
UN_LOOP(cosh, T, { W a = XR, b = XI; SETY(MF(cosh)(a) * MF(cos)(b), MF(sinh)(a) * MF(sin)(b)) })
UN_LOOP(tanh, T, { W a = 2 * XR, b = 2 * XI, r; r = 1. / (MF(cosh)(a) + MF(cos)(b)); SETY(MF(sinh)(a) * r, MF(sin)(b) * r) })
UN_LOOP(arcsin, T,
   {  W a = XR, b = XI, v1 = 1 - (a * a) + (b * b), v2 = -2 * a * b;
      W g = MF(sqrt)(MF(hypot)(v1, v2)), t = MF(atan2)(v2, v1) / 2;
      v1 = -b + g * MF(cos)(t); v2 = a + g * MF(sin)(t);
      SETY(MF(atan2)(v2, v1), MF(log)(v1 * v1 + v2 * v2) / -2)
   })
UN_LOOP(arccos, T,
   {  W a = XR, b = XI, v1 = 1 - (a * a) + (b * b), v2 = -2 * a * b;
      W g = MF(sqrt)(MF(hypot)(v1, v2)), t = MF(atan2)(v2, v1) / 2;
      v1 = a - g * MF(sin)(t); v2 = b + g * MF(cos)(t);
      SETY(MF(atan2)(v2, v1), MF(log)(v1 * v1 + v2 * v2) / -2)
   })
UN_LOOP(arctan, T,
   {  W a = XR, b = XI, v1 = (a * a), v2 = (b * b);
      y.real = FROMW(MF(atan2)(2 * a, 1 - v1 - v2) / 2);
      v2 = 1 + b;
      y.imag = FROMW(MF(log)(1 - 4 * b / (v2 * v2 + v1)) / -4);
   })
UN_LOOP(arcsinh, T,
   {  W a = XR, b = XI, v1 = 1 + (a * a) - (b * b), v2 = 2 * a * b;
      W g = MF(sqrt)(MF(hypot)(v1, v2)), t = MF(atan2)(v2, v1) / 2;
      v1 = a + g * MF(cos)(t); v2 = b + g * MF(sin)(t);
      SETY(MF(log)(v1 * v1 + v2 * v2) / 2, MF(atan2)(v2, v1))
   })
UN_LOOP(arccosh, T,
   {  W a = XR, b = XI, v1 = (a * a) - (b * b) - 1, v2 = 2 * a * b;
      W g = MF(sqrt)(MF(hypot)(v1, v2)), t = MF(atan2)(v2, v1) / 2;
      v1 = a + g * MF(cos)(t); v2 = b + g * MF(sin)(t);
      SETY(MF(log)(v1 * v1 + v2 * v2) / 2, MF(atan2)(v2, v1))
   })
/* arctanh: the reference writes both terms into the imaginary part and leaves the real
   part of the destination untouched (unary_ops.h:467-475); reproduced literally: the
   real part of y is whatever the destination held before. */
UN_LOOP(arctanh, T,
   {  W a = XR, b = XI, v1 = (a * a), v2 = (b * b);
      y = *(T *)q1;
      y.imag = FROMW(MF(atan2)(2 * b, 1 - v1 - v2) / 2);
      v1 = 1 - a;
      y.imag = FROMW(MF(log)(1 + 4 * a / (v1 * v1 + v2)) / 4);
   })
/* square root: Friedland's algorithm 312 (the CPU table uses this variant, template_unary.c:98) */
UN_LOOP(sqrt, T,
   {  W a = XR, b = XI, v = MF(hypot)(a, b);
      if (!(v > 0)) { y.real = FROMW(v); y.imag = y.real; }
      else if (isinf(b)) { y.real = HALF_OR_INF; y.imag = x.imag; }
      else if (isinf(a)) { y.real = FROMW((a > 0) ? a : 0); y.imag = FROMW(MF(copysign)((a < 0) ? a : 0, b)); }
      else if (a >= 0) { v = MF(sqrt)((a + v) * 0.5); y.real = FROMW(v); y.imag = FROMW(b / (2 * v)); }
      else { v = MF(sqrt)((-a + v) * 0.5); y.real = FROMW(((b >= 0) ? b : -b) / (2 * v)); y.imag = FROMW(MF(copysign)(v, b)); }
   })
UN_LOOP(cbrt, T,
   {  W a = XR, b = XI, s = ((a * a) + (b * b)), t;
      if (s > 0) { s = powf(s, 1. / 6); t = MF(atan2)(b, a) / 3; SETY(s * MF(cos)(t), s * MF(sin)(t)) }
      else { y.real = FROMW(0); y.imag = FROMW(0); }
   })
UN_LOOP(square, T, { W a = XR, b = XI; SETY(a * a - b * b, 2 * a * b) })
UN_LOOP(exp,   T, { W a = XR, b = XI, s = MF(exp)(a); SETY(s * MF(cos)(b), s * MF(sin)(b)) })
UN_LOOP(exp2,  T, { W a = XR, b = XI * ((W)0.69314718055994529), s = MF(exp2)(a); SETY(s * MF(cos)(b), s * MF(sin)(b)) })
UN_LOOP(exp10, T, { W a = XR, b = XI * ((W)2.3025850929940459), s = MF(exp)(((W)2.3025850929940459) * (a)); SETY(s * MF(cos)(b), s * MF(sin)(b)) })
UN_LOOP(expm1, T, { W a = XR, b = XI, s = MF(exp)(a); SETY(s * MF(cos)(b) - 1, s * MF(sin)(b)) })
UN_LOOP(log,   T, { W a = XR, b = XI, s = (a * a + b * b); SETY(MF(log)(s) * 0.5, MF(atan2)(b, a)) })
UN_LOOP(log2,  T, { W a = XR, b = XI, s = (a * a + b * b); SETY(MF(log2)(s) * 0.5, MF(atan2)(b, a) / ((W)0.69314718055994529)) })
UN_LOOP(log10, T, { W a = XR, b = XI, s = (a * a + b * b); SETY(MF(log10)(s) * 0.5, MF(atan2)(b, a) / ((W)2.3025850929940459)) })
UN_LOOP(log1p, T, { W a = XR + 1, b = XI, s = (a * a + b * b); SETY(MF(log)(s) * 0.5, MF(atan2)(b, a)) })
UN_LOOP(absolute, PT, y = FROMW(MF(hypot)(XR, XI));)
UN_LOOP(fabs, T, { y.real = FROMW(MF(hypot)(XR, XI)); y.imag = FROMW(0); })
UN_LOOP(sign, T,
   {  W a = XR, b = XI;
      if (isnan(a) || isnan(b)) y.real = FROMW(a + b);
      else { a = (((a > 0) - (a < 0)) + (a == 0) * ((b > 0) - (b < 0))); y.real = FROMW(a); }
      y.imag = FROMW(0);
   })
UN_LOOP(ceil,  T, SETY(MF(ceil)(XR),  MF(ceil)(XI)))
UN_LOOP(floor, T, SETY(MF(floor)(XR), MF(floor)(XI)))
UN_LOOP(trunc, T, SETY(MF(trunc)(XR), MF(trunc)(XI)))
UN_LOOP(round, T, SETY(MF(round)(XR), MF(round)(XI)))
UN_LOOP(isinf, o_bool, y = (isinf(XR) || isinf(XI)) ? 1 : 0;)
UN_LOOP(isnan, o_bool, y = (isnan(XR) || isinf(XI)) ? 1 : 0;)      /* imaginary part: isinf, as in the reference */
UN_LOOP(isfinite, o_bool, y = (isfinite(XR) && isfinite(XI)) ? 1 : 0;)
#undef XR
#undef XI
#undef YR
#undef YI
#undef SETZ
#undef SETY
#endif

#undef BIN_LOOP
#undef UN_LOOP
#undef PT
#undef TOW
#undef FROMW
#undef CAT
#undef CAT_
#undef CAT3
#undef CAT3_
