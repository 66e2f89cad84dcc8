/* Strided / broadcast elementwise engine for gfx950.
 *
 * Replaces the reference's elemwise1/2/3 kernel families and their host-side
 * analysers (solid/include/solid/core/gpu/apply_elemwise{1,2,3}.h,
 * solid/src/core/gpu/op/apply_elemwise{,1,2,3}.c). Design:
 *   - operands are normalised on the host: unit dimensions dropped, the
 *     destination's strides made positive and sorted ascending, mergeable
 *     dimensions merged, so that a contiguous tensor is one dimension;
 *   - one thread handles groups of VEC consecutive elements of dimension 0;
 *     operands whose dimension-0 stride equals their element size and whose
 *     addresses are 16-byte aligned use one <=128-bit access per group, other
 *     operands (strided, broadcast) use VEC element accesses;
 *   - the index of a group is decomposed with multiply-high division by
 *     invariant integers; one-dimensional problems need no division;
 *   - 32-bit group indices; larger tensors are cut on the host.
 */
#pragma once
#include <string.h>
#include "och_common.h"
#include "och_dtypes.h"

namespace och {

/* ---- division by an invariant 32-bit integer d >= 2 ---------------------- */
struct FastDiv { uint32_t d, m; uint16_t s1, s2; };

static inline FastDiv make_fastdiv(uint32_t d)
{  /* q = (t + ((n - t) >> s1)) >> s2 with t = mulhi(m, n), L = ceil(log2 d), m = floor(2^32 (2^L - d) / d) + 1,
      s1 = min(L, 1), s2 = max(L - 1, 0); exact for all 32-bit n and every d >= 1 (d = 1 gives m = 1, s1 = s2 = 0) */
   FastDiv f; f.d = d; f.m = 1; f.s1 = 0; f.s2 = 0;
   if (d < 2) return f;
   uint32_t L = 0; while ((1ull << L) < d) L++;
   f.m = (uint32_t)((((1ull << L) - d) << 32) / d + 1);
   f.s1 = 1; f.s2 = (uint16_t)(L - 1);
   return f;
}
OCH_HD uint32_t fastdiv(uint32_t n, const FastDiv &f)
{
#if defined(__HIP_DEVICE_COMPILE__)
   uint32_t t = __umulhi(f.m, n);
#else
   uint32_t t = (uint32_t)(((uint64_t)f.m * n) >> 32);
#endif
   return (t + ((n - t) >> f.s1)) >> f.s2;
}

/* ---- kernel parameters ---------------------------------------------------- */
template <int NOPS> struct EwParams
{
   char    *ptr[NOPS];
   int64_t  gstride[NOPS];                 /* byte step of one group (VEC elements) along dim 0 */
   int64_t  estride[NOPS];                 /* byte step of one element along dim 0 */
   int64_t  stride[NOPS][OCH_MAX_DIMS];    /* byte strides of dims 1.. (index 0 unused) */
   FastDiv  div[OCH_MAX_DIMS];             /* div[0]: groups along dim 0, div[d]: size of dim d */
   uint32_t ngroups;                       /* total number of groups */
   uint64_t group0;                        /* first flat element index (for index-dependent ops) */
   int      ndims;
   int      vecmode[NOPS];
   int      nt;                            /* streaming launch: wide accesses carry the nontemporal hint */
   uint32_t unr;                           /* groups per thread of this launch (at most the kernel's UNR) */
   uint32_t block;                         /* threads per workgroup of this launch */
   uint64_t row_n0;                        /* row kernels: elements in a row of dimension 0 (div[0] then divides by the chunks of a row) */
};

template <class T, int VEC> struct alignas((sizeof(T) * VEC) > 16 ? 16 : (sizeof(T) * VEC)) Pack { T v[VEC]; };

template <class T> constexpr int vec_for_c() { return (16 / (int)sizeof(T)) > 0 ? (16 / (int)sizeof(T)) : 1; }

/* Wide accesses go through a native vector type of the pack's byte width, so that the compiler
   keeps them as ONE load/store instruction (an aggregate copy is split into element accesses
   and may then be merged with the strided path into element-wise loads). */
typedef unsigned int och_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int och_u32x4 __attribute__((ext_vector_type(4)));
template <int BYTES> struct RawVec;
template <> struct RawVec<1>  { typedef uint8_t  type; };
template <> struct RawVec<2>  { typedef uint16_t type; };
template <> struct RawVec<4>  { typedef uint32_t type; };
template <> struct RawVec<8>  { typedef och_u32x2 type; };
template <> struct RawVec<16> { typedef och_u32x4 type; };

/* nt (a compile-time constant at every call site: a run-time choice between the two forms is folded into the
   plain one): nontemporal hint for data that is touched once (large streaming launches); measured on MI355X,
   a float64 add of 3 x 134 MB runs at 6.4 TB/s with the hint and one group per thread, 5.4 TB/s without */
template <class T, int VEC, bool NT = false>
OCH_D void load_wide(Pack<T, VEC> &p, const char *addr)
{
   static_assert(sizeof(Pack<T, VEC>) <= 16, "pack wider than 128 bits");
   typedef typename RawVec<sizeof(Pack<T, VEC>)>::type V;
   V raw;
   if constexpr (NT) raw = __builtin_nontemporal_load(reinterpret_cast<const V *>(addr));
   else    raw = *reinterpret_cast<const V *>(addr);
   __builtin_memcpy(&p, &raw, sizeof(V));
}
template <class T, int VEC, bool NT = false>
OCH_D void store_wide(const Pack<T, VEC> &p, char *addr)
{
   typedef typename RawVec<sizeof(Pack<T, VEC>)>::type V;
   V raw;
   __builtin_memcpy(&raw, &p, sizeof(V));
   if constexpr (NT) __builtin_nontemporal_store(raw, reinterpret_cast<V *>(addr));
   else    *reinterpret_cast<V *>(addr) = raw;
}

/* A pack read from an address that is only aligned to its element: one load instruction all the same (the device runs
   with unaligned access enabled; the under-aligned vector type tells the compiler not to assume more). */
template <class T, int VEC, bool NT = false>
OCH_D void load_unaligned(Pack<T, VEC> &p, const char *addr)
{
   typedef typename RawVec<sizeof(Pack<T, VEC>)>::type V;
   typedef V __attribute__((aligned(alignof(T) < sizeof(V) ? alignof(T) : sizeof(V)))) VU;
   V raw;
   if constexpr (NT) raw = __builtin_nontemporal_load(reinterpret_cast<const VU *>(addr));
   else    raw = *reinterpret_cast<const VU *>(addr);
   __builtin_memcpy(&p, &raw, sizeof(V));
}

/* Source elements one apart (a step-2 slice along the first dimension): the 2 VEC consecutive elements that hold the
   group are read with one or two <=128-bit loads and every second one is kept. The element behind the last one kept
   lies in the same aligned 16-byte unit as an element of the tensor, so no load leaves such a unit. Measured on MI355X
   for int16 (step 2) -> float32: 4.8 TB/s of the bytes asked for against 4.6 with one 2-byte load per element (the
   memory system moves the skipped elements either way: 8 bytes of traffic for 6 bytes asked for). */
template <class T, int VEC, bool NT = false>
OCH_D void load_even(Pack<T, VEC> &p, const char *addr)
{
   constexpr int SPAN = 2 * VEC * (int)sizeof(T);
   constexpr int W = SPAN > 16 ? 16 : SPAN, NL = SPAN / W;
   typedef typename RawVec<W>::type V;
   V raw[NL];
#pragma unroll
   for (int l = 0; l < NL; l++)
   {  if constexpr (NT) raw[l] = __builtin_nontemporal_load(reinterpret_cast<const V *>(addr) + l);
      else    raw[l] = reinterpret_cast<const V *>(addr)[l];
   }
   T e[2 * VEC];
   __builtin_memcpy(e, raw, SPAN);
#pragma unroll
   for (int k = 0; k < VEC; k++) p.v[k] = e[2 * k];
}
template <class T, int VEC> constexpr bool even_loads_pay() { return VEC > 1 && sizeof(T) <= 4; }

/* vec: 1 = one wide access, 2 = every second of 2 VEC consecutive elements (inputs only), 0 = element accesses */
template <class T, int VEC, bool NT = false>
OCH_D void load_pack(Pack<T, VEC> &p, const char *addr, int64_t estride, int vec)
{
   if (vec == 1) load_wide<T, VEC, NT>(p, addr);
   else if (even_loads_pay<T, VEC>() && vec == 2)
   {  if constexpr (even_loads_pay<T, VEC>()) load_even<T, VEC, NT>(p, addr); }
   else if (estride == 0)
   {  /* broadcast along the vector: one load serves all elements */
      const T x = *reinterpret_cast<const T *>(addr);
#pragma unroll
      for (int k = 0; k < VEC; k++) p.v[k] = x;
   }
   else
   {
#pragma unroll
      for (int k = 0; k < VEC; k++) p.v[k] = *reinterpret_cast<const T *>(addr + k * estride);
   }
}
/* load_pack in two steps for kernels that issue their loads long before they use them: a broadcast along the vector is
   one load into the first element, and copying it to the others -- which has to wait for the load, and with it for
   every load issued before -- is left to load_pack_finish at the point of use */
template <class T, int VEC, bool NT = false>
OCH_D void load_pack_issue(Pack<T, VEC> &p, const char *addr, int64_t estride, int vec)
{
   if (vec == 0 && estride == 0) p.v[0] = *reinterpret_cast<const T *>(addr);
   else load_pack<T, VEC, NT>(p, addr, estride, vec);
}
template <class T, int VEC>
OCH_D void load_pack_finish(Pack<T, VEC> &p, int64_t estride, int vec)
{
   if (vec == 0 && estride == 0)
   {
#pragma unroll
      for (int k = 1; k < VEC; k++) p.v[k] = p.v[0];
   }
}

template <class T, int VEC, bool NT = false>
OCH_D void store_pack(const Pack<T, VEC> &p, char *addr, int64_t estride, int vec)
{
   if (vec) store_wide<T, VEC, NT>(p, addr);
   else
   {
#pragma unroll
      for (int k = 0; k < VEC; k++) *reinterpret_cast<T *>(addr + k * estride) = p.v[k];
   }
}

template <int NOPS>
OCH_D void group_offsets(const EwParams<NOPS> &p, uint32_t g, int64_t (&off)[NOPS])
{
   if (p.ndims == 1)
   {
#pragma unroll
      for (int k = 0; k < NOPS; k++) off[k] = (int64_t)g * p.gstride[k];
   }
   else
   {  uint32_t q = fastdiv(g, p.div[0]);
      uint32_t i = g - q * p.div[0].d;
#pragma unroll
      for (int k = 0; k < NOPS; k++) off[k] = (int64_t)i * p.gstride[k];
      for (int d = 1; d < p.ndims - 1; d++)
      {  uint32_t q2 = fastdiv(q, p.div[d]);
         i = q - q2 * p.div[d].d; q = q2;
#pragma unroll
         for (int k = 0; k < NOPS; k++) off[k] += (int64_t)i * p.stride[k][d];
      }
#pragma unroll
      for (int k = 0; k < NOPS; k++) off[k] += (int64_t)q * p.stride[k][p.ndims - 1];
   }
}

/* A wave of these kernels lives for one or two memory round trips, so what it does before its first load counts. Left
   to itself the compiler fetches every kernel argument where it is first used: four dependent scalar-load round trips
   before the first global load of the one-dimensional path. Naming the fields that every path needs in an empty asm at
   the top of the kernel makes it fetch them together, one round trip (float64 <- int32 cast of 2^24 elements on
   MI355X: 5.97 -> 6.3 TB/s). */
template <int NOPS>
OCH_D void ew_fetch_arguments(const EwParams<NOPS> &p)
{
#pragma unroll
   for (int k = 0; k < NOPS; k++) asm volatile("" :: "s"(p.ptr[k]), "s"(p.gstride[k]));
   asm volatile("" :: "s"(p.ngroups), "s"(p.ndims), "s"(p.unr), "s"(p.block));
}

#define OCH_EW_BLOCK 256
/* workgroup size of streaming launches of the all-wide kernels: on MI355X a float64 add of 3 x 134 MB runs at 6.43 TB/s
   with 512 threads per workgroup and at 6.38 with 256, a float32 -> float64 cast at 6.28 against 6.18 */
#define OCH_EW_BLOCK_STREAM 512
#define OCH_EW_MAX_BLOCK 512
/* launches that move at least this many bytes are treated as streaming (larger than the L2 of all XCDs) */
#define OCH_EW_STREAM_BYTES (48ull << 20)

/* z = f(x, y) */
template <class F, int VEC, int UNR, bool FAST, bool NT = false>
__global__ __launch_bounds__(OCH_EW_MAX_BLOCK) void ew3_kernel(const EwParams<3> p)
{
   typedef typename F::A A; typedef typename F::B B; typedef typename F::R R;
   ew_fetch_arguments<3>(p);
   const uint32_t base = blockIdx.x * (p.block * p.unr) + threadIdx.x;
   Pack<A, VEC> a[UNR]; Pack<B, VEC> b[UNR]; int64_t off[UNR][3];
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  uint32_t g = base + u * p.block;
      if ((uint32_t)u < p.unr && g < p.ngroups)
      {  group_offsets<3>(p, g, off[u]);
         load_pack<A, VEC, NT>(a[u], p.ptr[0] + off[u][0], p.estride[0], FAST ? 1 : p.vecmode[0]);
         load_pack<B, VEC, NT>(b[u], p.ptr[1] + off[u][1], p.estride[1], FAST ? 1 : p.vecmode[1]);
      }
   }
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  uint32_t g = base + u * p.block;
      if ((uint32_t)u < p.unr && g < p.ngroups)
      {  Pack<R, VEC> r;
#pragma unroll
         for (int k = 0; k < VEC; k++) r.v[k] = F::f(a[u].v[k], b[u].v[k]);
         store_pack<R, VEC, NT>(r, p.ptr[2] + off[u][2], p.estride[2], FAST ? 1 : p.vecmode[2]);
      }
   }
}

/* y = f(x) */
template <class F, int VEC, int UNR, bool FAST, bool NT = false>
__global__ __launch_bounds__(OCH_EW_MAX_BLOCK) void ew2_kernel(const EwParams<2> p)
{
   typedef typename F::A A; typedef typename F::R R;
   ew_fetch_arguments<2>(p);
   const uint32_t base = blockIdx.x * (p.block * p.unr) + threadIdx.x;
   Pack<A, VEC> a[UNR]; int64_t off[UNR][2];
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  uint32_t g = base + u * p.block;
      if ((uint32_t)u < p.unr && g < p.ngroups)
      {  group_offsets<2>(p, g, off[u]);
         load_pack<A, VEC, NT>(a[u], p.ptr[0] + off[u][0], p.estride[0], FAST ? 1 : p.vecmode[0]);
      }
   }
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  uint32_t g = base + u * p.block;
      if ((uint32_t)u < p.unr && g < p.ngroups)
      {  Pack<R, VEC> r;
#pragma unroll
         for (int k = 0; k < VEC; k++) r.v[k] = F::f(a[u].v[k]);
         store_pack<R, VEC, NT>(r, p.ptr[1] + off[u][1], p.estride[1], FAST ? 1 : p.vecmode[1]);
      }
   }
}

/* x = f(x, flat index, param): fill, conditional fill, steps. F::RMW tells whether the
   old value is read. The flat index counts elements in the order of the NORMALISED
   dimensions, so index-dependent functors are launched without reordering. */
template <class F, int VEC, int UNR, bool FAST, bool NT = false>
__global__ __launch_bounds__(OCH_EW_MAX_BLOCK) void ew1_kernel(const EwParams<1> p, const typename F::Param prm)
{
   typedef typename F::R R;
   ew_fetch_arguments<1>(p);
   const uint32_t base = blockIdx.x * (p.block * p.unr) + threadIdx.x;
#pragma unroll
   for (int u = 0; u < UNR; u++)
   {  uint32_t g = base + u * p.block;
      if ((uint32_t)u < p.unr && g < p.ngroups)
      {  int64_t off[1];
         group_offsets<1>(p, g, off);
         Pack<R, VEC> r;
         if constexpr (F::RMW) load_pack<R, VEC>(r, p.ptr[0] + off[0], p.estride[0], FAST ? 1 : p.vecmode[0]);
#pragma unroll
         for (int k = 0; k < VEC; k++) r.v[k] = F::f(r.v[k], p.group0 + (uint64_t)g * VEC + k, prm);
         store_pack<R, VEC, NT>(r, p.ptr[0] + off[0], p.estride[0], FAST ? 1 : p.vecmode[0]);
      }
   }
}


/* ---- row kernels: unit-stride rows that are not whole aligned vectors ----------
   A sub-matrix whose width is not a multiple of VEC, whose rows start inside a 16-byte unit or whose pitch is not a
   multiple of 16 bytes cannot take the all-wide kernels, and with one element per thread 1- and 2-byte types move a
   byte or two per lane and instruction. Here a work item is one ALIGNED unit of a destination row (VEC elements,
   WD = VEC * sizeof(R) <= 16 bytes): units that lie inside the row are written with one wide store, and their inputs are
   read with one load each from wherever the same elements lie in the input rows (aligned to the element only); the
   units at the two ends of a row hold fewer elements and move them one by one, so no byte outside a row is ever
   written, nor read. Every row gets the number of units of the worst-placed row; units left over do nothing.
   Inputs that are not unit-stride along the row (a broadcast, a stepped or transposed view) are read element by
   element (vecmode 0). */
/* Unit c of a destination row of n0 elements of esr bytes that starts m bytes into an aligned unit of `vec` elements:
   row position e0 of the unit's element 0 (negative in the first unit when m > 0) and the range [lo, hi) of its
   elements that lie inside the row; false when there are none. */
__host__ __device__ inline bool row_unit_range(uint32_t c, int m, int esr, int vec, uint64_t n0, int64_t &e0, int &lo, int &hi)
{
   e0 = (int64_t)c * vec - m / esr;
   const int64_t left = (int64_t)n0 - e0;
   lo = (e0 < 0) ? (int)(-e0) : 0;
   hi = (left >= vec) ? vec : (left > 0 ? (int)left : 0);
   return hi > lo;
}
/* units every row is given: those of a row that starts on the last element of an aligned unit */
static inline uint64_t row_units(uint64_t n0, int esr, int vec)
{  const uint64_t wd = (uint64_t)vec * esr;
   return (wd - esr + n0 * esr + wd - 1) / wd;
}

template <int NOPS>
OCH_D bool row_unit(const EwParams<NOPS> &p, uint32_t g, int wd, int esr, int vec, int64_t (&off)[NOPS], int64_t &e0, int &lo, int &hi)
{
   const uint32_t r = fastdiv(g, p.div[0]), c = g - r * p.div[0].d;
#pragma unroll
   for (int k = 0; k < NOPS; k++) off[k] = 0;
   uint32_t q = r;
   for (int d = 1; d < p.ndims - 1; d++)
   {  const uint32_t q2 = fastdiv(q, p.div[d]), i = q - q2 * p.div[d].d; q = q2;
#pragma unroll
      for (int k = 0; k < NOPS; k++) off[k] += (int64_t)i * p.stride[k][d];
   }
   if (p.ndims > 1)
   {
#pragma unroll
      for (int k = 0; k < NOPS; k++) off[k] += (int64_t)q * p.stride[k][p.ndims - 1];
   }
   const int m = (int)((uintptr_t)(p.ptr[NOPS - 1] + off[NOPS - 1]) & (uintptr_t)(wd - 1));    /* bytes of the first unit in front of the row */
   return row_unit_range(c, m, esr, vec, p.row_n0, e0, lo, hi);
}

template <class F, int VEC, bool NT = false>
__global__ __launch_bounds__(OCH_EW_BLOCK) void ew3_rows_kernel(const EwParams<3> p)
{
   typedef typename F::A A; typedef typename F::B B; typedef typename F::R R;
   const uint32_t g = blockIdx.x * OCH_EW_BLOCK + threadIdx.x;
   if (g >= p.ngroups) return;
   int64_t off[3], e0; int lo, hi;
   if (!row_unit<3>(p, g, VEC * (int)sizeof(R), (int)sizeof(R), VEC, off, e0, lo, hi)) return;
   const char *pa = p.ptr[0] + off[0] + e0 * p.estride[0], *pb = p.ptr[1] + off[1] + e0 * p.estride[1];
   char *pr = p.ptr[2] + off[2] + e0 * (int64_t)sizeof(R);
   if (lo == 0 && hi == VEC)
   {  Pack<A, VEC> a; Pack<B, VEC> b; Pack<R, VEC> r;
      if (p.vecmode[0]) load_unaligned<A, VEC, NT>(a, pa); else load_pack<A, VEC>(a, pa, p.estride[0], 0);
      if (p.vecmode[1]) load_unaligned<B, VEC, NT>(b, pb); else load_pack<B, VEC>(b, pb, p.estride[1], 0);
#pragma unroll
      for (int k = 0; k < VEC; k++) r.v[k] = F::f(a.v[k], b.v[k]);
      store_wide<R, VEC, NT>(r, pr);
   }
   else
   {  for (int k = lo; k < hi; k++)
         *reinterpret_cast<R *>(pr + k * (int64_t)sizeof(R)) =
            F::f(*reinterpret_cast<const A *>(pa + k * p.estride[0]), *reinterpret_cast<const B *>(pb + k * p.estride[1]));
   }
}

template <class F, int VEC, bool NT = false>
__global__ __launch_bounds__(OCH_EW_BLOCK) void ew2_rows_kernel(const EwParams<2> p)
{
   typedef typename F::A A; typedef typename F::R R;
   const uint32_t g = blockIdx.x * OCH_EW_BLOCK + threadIdx.x;
   if (g >= p.ngroups) return;
   int64_t off[2], e0; int lo, hi;
   if (!row_unit<2>(p, g, VEC * (int)sizeof(R), (int)sizeof(R), VEC, off, e0, lo, hi)) return;
   const char *pa = p.ptr[0] + off[0] + e0 * p.estride[0];
   char *pr = p.ptr[1] + off[1] + e0 * (int64_t)sizeof(R);
   if (lo == 0 && hi == VEC)
   {  Pack<A, VEC> a; Pack<R, VEC> r;
      if (p.vecmode[0]) load_unaligned<A, VEC, NT>(a, pa); else load_pack<A, VEC>(a, pa, p.estride[0], 0);
#pragma unroll
      for (int k = 0; k < VEC; k++) r.v[k] = F::f(a.v[k]);
      store_wide<R, VEC, NT>(r, pr);
   }
   else
   {  for (int k = lo; k < hi; k++)
         *reinterpret_cast<R *>(pr + k * (int64_t)sizeof(R)) = F::f(*reinterpret_cast<const A *>(pa + k * p.estride[0]));
   }
}

/* x = f(x, flat index, param) on rows: the flat index of an element is its row times the row length plus its position */
template <class F, int VEC, bool NT = false>
__global__ __launch_bounds__(OCH_EW_BLOCK) void ew1_rows_kernel(const EwParams<1> p, const typename F::Param prm)
{
   typedef typename F::R R;
   const uint32_t g = blockIdx.x * OCH_EW_BLOCK + threadIdx.x;
   if (g >= p.ngroups) return;
   int64_t off[1], e0; int lo, hi;
   if (!row_unit<1>(p, g, VEC * (int)sizeof(R), (int)sizeof(R), VEC, off, e0, lo, hi)) return;
   char *pr = p.ptr[0] + off[0] + e0 * (int64_t)sizeof(R);
   const uint64_t flat = p.group0 + (uint64_t)fastdiv(g, p.div[0]) * p.row_n0 + (uint64_t)e0;     /* of element 0 of the unit (wraps back for k >= lo) */
   if (lo == 0 && hi == VEC)
   {  Pack<R, VEC> r;
      if constexpr (F::RMW) load_wide<R, VEC>(r, pr);
#pragma unroll
      for (int k = 0; k < VEC; k++) r.v[k] = F::f(r.v[k], flat + k, prm);
      store_wide<R, VEC, NT>(r, pr);
   }
   else
   {  for (int k = lo; k < hi; k++)
      {  R x{};
         if constexpr (F::RMW) x = *reinterpret_cast<const R *>(pr + k * (int64_t)sizeof(R));
         *reinterpret_cast<R *>(pr + k * (int64_t)sizeof(R)) = F::f(x, flat + k, prm);
      }
   }
}


/* ---- tiled kernels for transposed operands ----------------------------------
   When an input is contiguous along a dimension other than the output's fastest one (a
   transposed view), reading it in output order touches one element per cache line. These
   kernels work on TILE x TILE blocks of (dimension 0, dimension d1): such an input is read
   with 128-bit loads along d1, parked transposed in LDS, and then consumed in output order;
   the other operands are accessed directly along dimension 0. */
/* threads per tile: a 64 x 64 tile of 8-byte elements takes 33 KB of LDS, so workgroups of 256 threads leave a compute
   unit with 16 waves; 1024 threads per tile (two 16-byte loads in flight per thread instead of eight) fill it with 32
   (transposed float64 add, 4096 x 4096, on MI355X: 5.9 -> 6.2 TB/s). The smaller tiles of the other types fit eight times
   with 256 threads. */
constexpr int tile_threads(size_t maxsize) { return maxsize == 8 ? 1024 : 256; }
template <int NOPS> struct TileParams
{  /* the fields every workgroup reads come first, so that one scalar load brings them in (see tile_fetch_arguments) */
   char    *ptr[NOPS];
   int64_t  s0[NOPS], s1[NOPS];             /* byte strides along dimension 0 and along d1 */
   uint32_t n0, n1;                         /* extents of dimension 0 and d1 */
   int      nouter;
   int      trans[NOPS];                    /* read through LDS */
   int      vecmode[NOPS];                  /* direct access may use VEC-wide loads/stores */
   int      lds_off[NOPS];                  /* byte offset of the operand's LDS tile */
   int      nt;                             /* streaming launch: nontemporal hint on global accesses */
   int      diagonal;                       /* walk the tile grid along diagonals (see tile_row) */
   FastDiv  rowdiv;                         /* division by the number of tile rows (gridDim.y) */
   int64_t  so[NOPS][OCH_MAX_DIMS];         /* byte strides of the remaining (outer) dimensions */
   FastDiv  odiv[OCH_MAX_DIMS];
};

/* one scalar-load round trip for the arguments instead of one per first use (see ew_fetch_arguments) */
template <int NOPS>
OCH_D void tile_fetch_arguments(const TileParams<NOPS> &p)
{
#pragma unroll
   for (int k = 0; k < NOPS; k++) asm volatile("" :: "s"(p.ptr[k]), "s"(p.s0[k]), "s"(p.s1[k]), "s"(p.trans[k]), "s"(p.vecmode[k]), "s"(p.lds_off[k]));
   asm volatile("" :: "s"(p.n0), "s"(p.n1), "s"(p.nouter), "s"(p.diagonal), "s"(p.rowdiv.d), "s"(p.rowdiv.m), "s"(p.rowdiv.s1), "s"(p.rowdiv.s2));
}

constexpr int tile_dim(size_t maxsize) { return maxsize >= 16 ? 32 : 64; }
template <class T> constexpr int tile_pitch(int tile) { return tile + (sizeof(T) >= 4 ? 1 : 4 / (int)sizeof(T)); }
template <class T> constexpr int tile_bytes(int tile) { return ((tile * tile_pitch<T>(tile) * (int)sizeof(T)) + 15) / 16 * 16; }

/* Byte offset of position (i0, i1) within a tile. The host takes the tiled kernels only when every stride along the two
   tile dimensions is below 2^23 bytes in magnitude, so 24-bit multiplies and 32-bit sums are exact: a handful of
   full-rate instructions per address where 64-bit products cost several quarter-rate ones (with 32 waves per compute
   unit that arithmetic was a fifth of a tile's time). */
OCH_D int64_t tile_offset(uint32_t i0, int s0, uint32_t i1, int s1) { return (int64_t)(__mul24((int)i0, s0) + __mul24((int)i1, s1)); }

/* Loads of positions outside an edge tile are not skipped but redirected to a position inside it (and what they
   bring is never used): without a branch around them the compiler issues all loads of a thread back to back before
   the first one is waited for. n1 is a multiple of the vector length (the host checks it), n0 >= 1.
   tile_load issues the loads of one thread, tile_park writes what they brought into the LDS tile, transposed. */
template <class T, int TILE, int THREADS> struct TileStage
{
   static constexpr int VK = vec_for_c<T>();
   static constexpr int LPR = TILE / VK;                        /* lanes per row (fixed index along dimension 0) */
   static constexpr int RPP = THREADS / LPR;                    /* rows per pass */
   static constexpr int PASSES = (TILE + RPP - 1) / RPP;
   static constexpr int PITCH = tile_pitch<T>(TILE);
   Pack<T, VK> v[PASSES];
   template <bool NT> OCH_D void load(const char *base, int s0, uint32_t n0, uint32_t n1)
   {  const uint32_t i1 = (threadIdx.x % LPR) * VK, row = threadIdx.x / LPR;
      const uint32_t i1c = (i1 < n1) ? i1 : 0;
#pragma unroll
      for (int u = 0; u < PASSES; u++)
      {  const uint32_t i0 = row + u * RPP, i0c = (i0 < n0) ? i0 : n0 - 1;
         load_wide<T, VK, NT>(v[u], base + tile_offset(i0c, s0, i1c, (int)sizeof(T)));
      }
   }
   OCH_D void park(T *lds) const
   {  const uint32_t i1 = (threadIdx.x % LPR) * VK, row = threadIdx.x / LPR;
#pragma unroll
      for (int u = 0; u < PASSES; u++)
      {  const uint32_t i0 = row + u * RPP;
         if (PASSES * RPP <= TILE || i0 < (uint32_t)TILE)
         {
#pragma unroll
            for (int j = 0; j < VK; j++) lds[(i1 + j) * PITCH + i0] = v[u].v[j];
         }
      }
   }
};

/* Tile row of a block. Blocks that run together have neighbouring blockIdx.x. When the pitch of the transposed operand
   is a power of two between 16 KB and 64 KB (4096 x 4096 or 8192 x 8192 float64), the straight order makes them all read
   the same 512-byte column of that operand at a pitch of one matrix row, i.e. the same few memory channels; shifting
   the tile row by (three times) the tile column walks the grid along diagonals and spreads both the reads and the writes
   (measured on MI355X: 6.2 against 5.6 TB/s at 4096 x 4096; a shift of one tile row per column gives 6.15, square
   super-tiles of 4 to 32 tiles 5.7 - 5.9). For every other pitch the straight order is the faster one by
   10 - 25 % (5.5 against 4.4 TB/s at 4224 x 4224), so the host chooses per launch.
   What a wave computes before its first load is scalar work that the waves of a SIMD do one after the other, so it
   is kept short: the remainder comes from a multiply-shift division prepared on the host, the tile origins from
   32 x 32 -> 64-bit products (the host keeps tile coordinates below 2^31 and strides below 2^23). */
template <int NOPS>
OCH_D uint32_t tile_row(const TileParams<NOPS> &p)
{  if (!p.diagonal) return blockIdx.y;
   const uint32_t t = blockIdx.y + 3 * blockIdx.x;
   return t - fastdiv(t, p.rowdiv) * p.rowdiv.d;
}

template <int NOPS>
OCH_D void tile_origin(const TileParams<NOPS> &p, int tile, uint32_t trow, int64_t (&off)[NOPS])
{
   uint32_t q = blockIdx.z;
#pragma unroll
   for (int k = 0; k < NOPS; k++)
      off[k] = (int64_t)(int)(blockIdx.x * tile) * (int64_t)(int)p.s0[k] + (int64_t)(int)(trow * tile) * (int64_t)(int)p.s1[k];
   for (int d = 0; d < p.nouter; d++)
   {  uint32_t q2 = fastdiv(q, p.odiv[d]);
      uint32_t i = q - q2 * p.odiv[d].d; q = q2;
#pragma unroll
      for (int k = 0; k < NOPS; k++) off[k] += (int64_t)i * p.so[k][d];
   }
}

template <class A, class B, class R> constexpr size_t max_size3()
{  return sizeof(A) > sizeof(B) ? (sizeof(A) > sizeof(R) ? sizeof(A) : sizeof(R)) : (sizeof(B) > sizeof(R) ? sizeof(B) : sizeof(R)); }

template <class F, int VEC, bool NT>
__global__ __launch_bounds__(tile_threads(max_size3<typename F::A, typename F::B, typename F::R>())) void ew3_tile_kernel(const TileParams<3> p)
{
   typedef typename F::A A; typedef typename F::B B; typedef typename F::R R;
   constexpr size_t MAXS = max_size3<A, B, R>();
   constexpr int TILE = tile_dim(MAXS), THREADS = tile_threads(MAXS);
   extern __shared__ __align__(16) char och_tile_lds[];
   tile_fetch_arguments<3>(p);
   A *la = reinterpret_cast<A *>(och_tile_lds + p.lds_off[0]);
   B *lb = reinterpret_cast<B *>(och_tile_lds + p.lds_off[1]);
   int64_t off[3];
   const uint32_t trow = tile_row(p);
   tile_origin<3>(p, TILE, trow, off);
   const uint32_t r0 = p.n0 - blockIdx.x * TILE, r1 = p.n1 - trow * TILE;
   const uint32_t n0 = r0 < (uint32_t)TILE ? r0 : TILE, n1 = r1 < (uint32_t)TILE ? r1 : TILE;
   /* order of a workgroup: loads of the transposed operands, loads of the operands that are read straight from memory
      (their latency runs in parallel instead of starting behind the barrier), LDS, barrier, LDS */
   constexpr int LPC = TILE / VEC, CPP = THREADS / LPC, PASSES = (TILE + CPP - 1) / CPP;
   const uint32_t i0 = (threadIdx.x % LPC) * VEC, col = threadIdx.x / LPC;
   const uint32_t i0c = (i0 < n0) ? i0 : 0;                  /* n0 is a multiple of VEC */
   TileStage<A, TILE, THREADS> sa; TileStage<B, TILE, THREADS> sb;
   Pack<A, VEC> a[PASSES]; Pack<B, VEC> b[PASSES];
   if (p.trans[0]) sa.template load<NT>(p.ptr[0] + off[0], (int)p.s0[0], n0, n1);
   if (p.trans[1]) sb.template load<NT>(p.ptr[1] + off[1], (int)p.s0[1], n0, n1);
#pragma unroll
   for (int u = 0; u < PASSES; u++)
   {  const uint32_t i1 = col + u * CPP, i1c = (i1 < n1) ? i1 : n1 - 1;
      if (!p.trans[0]) load_pack_issue<A, VEC, NT>(a[u], p.ptr[0] + off[0] + tile_offset(i0c, (int)p.s0[0], i1c, (int)p.s1[0]), p.s0[0], p.vecmode[0]);
      if (!p.trans[1]) load_pack_issue<B, VEC, NT>(b[u], p.ptr[1] + off[1] + tile_offset(i0c, (int)p.s0[1], i1c, (int)p.s1[1]), p.s0[1], p.vecmode[1]);
   }
   if (p.trans[0]) sa.park(la);
   if (p.trans[1]) sb.park(lb);
   __syncthreads();
   /* every load of this thread was issued before the barrier; waiting for all of them here, in one place that every
      path runs through, lets the compiler see that nothing is outstanding afterwards. Otherwise the paths through
      the run-time operand modes merge with different numbers of loads in flight, it falls back to waiting for
      everything -- stores included -- in front of each later pass, and a thread's second store waits for its first
      to be acknowledged (transposed float64 add 4096 x 4096: 5.85 -> 6.2 TB/s) */
   __builtin_amdgcn_s_waitcnt(0x0F70);          /* vmcnt(0); expcnt and lgkmcnt left alone */
#pragma unroll
   for (int u = 0; u < PASSES; u++)
   {  const uint32_t i1 = col + u * CPP, i1c = (i1 < n1) ? i1 : n1 - 1;
      if (p.trans[0])
      {
#pragma unroll
         for (int k = 0; k < VEC; k++) a[u].v[k] = la[i1c * tile_pitch<A>(TILE) + i0c + k];
      }
      else load_pack_finish<A, VEC>(a[u], p.s0[0], p.vecmode[0]);
      if (p.trans[1])
      {
#pragma unroll
         for (int k = 0; k < VEC; k++) b[u].v[k] = lb[i1c * tile_pitch<B>(TILE) + i0c + k];
      }
      else load_pack_finish<B, VEC>(b[u], p.s0[1], p.vecmode[1]);
   }
#pragma unroll
   for (int u = 0; u < PASSES; u++)
   {  const uint32_t i1 = col + u * CPP;
      if (i0 < n0 && i1 < n1)
      {  Pack<R, VEC> r;
#pragma unroll
         for (int k = 0; k < VEC; k++) r.v[k] = F::f(a[u].v[k], b[u].v[k]);
         store_pack<R, VEC, NT>(r, p.ptr[2] + off[2] + tile_offset(i0, (int)p.s0[2], i1, (int)p.s1[2]), p.s0[2], p.vecmode[2]);
      }
   }
}

template <class F, int VEC, bool NT>
__global__ __launch_bounds__(tile_threads(max_size3<typename F::A, typename F::A, typename F::R>())) void ew2_tile_kernel(const TileParams<2> p)
{
   typedef typename F::A A; typedef typename F::R R;
   constexpr size_t MAXS = sizeof(A) > sizeof(R) ? sizeof(A) : sizeof(R);
   constexpr int TILE = tile_dim(MAXS), THREADS = tile_threads(MAXS);
   extern __shared__ __align__(16) char och_tile_lds[];
   tile_fetch_arguments<2>(p);
   A *la = reinterpret_cast<A *>(och_tile_lds);
   int64_t off[2];
   const uint32_t trow = tile_row(p);
   tile_origin<2>(p, TILE, trow, off);
   const uint32_t r0 = p.n0 - blockIdx.x * TILE, r1 = p.n1 - trow * TILE;
   const uint32_t n0 = r0 < (uint32_t)TILE ? r0 : TILE, n1 = r1 < (uint32_t)TILE ? r1 : TILE;
   TileStage<A, TILE, THREADS> sa;
   sa.template load<NT>(p.ptr[0] + off[0], (int)p.s0[0], n0, n1);
   sa.park(la);
   __syncthreads();
   constexpr int LPC = TILE / VEC, CPP = THREADS / LPC, PASSES = (TILE + CPP - 1) / CPP;
   const uint32_t i0 = (threadIdx.x % LPC) * VEC, col = threadIdx.x / LPC;
   const uint32_t i0c = (i0 < n0) ? i0 : 0;
#pragma unroll
   for (int u = 0; u < PASSES; u++)
   {  const uint32_t i1 = col + u * CPP, i1c = (i1 < n1) ? i1 : n1 - 1;
      Pack<R, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; k++) r.v[k] = F::f(la[i1c * tile_pitch<A>(TILE) + i0c + k]);
      if (i0 < n0 && i1 < n1)
         store_pack<R, VEC, NT>(r, p.ptr[1] + off[1] + tile_offset(i0, (int)p.s0[1], i1, (int)p.s1[1]), p.s0[1], p.vecmode[1]);
   }
}

/* ---- host side: normalisation --------------------------------------------- */
template <int NOPS> struct EwShape
{
   int      ndims;
   uint64_t size[OCH_MAX_DIMS];
   int64_t  stride[NOPS][OCH_MAX_DIMS];
   char    *ptr[NOPS];
   uint64_t nelem;
};

/* key: operand whose strides drive sorting (the destination). reorder=false keeps the
   caller's dimension order and stride signs (needed when the flat index matters).
   Returns -1 on bad input. */
template <int NOPS>
static int ew_normalize(EwShape<NOPS> &s, int ndims, const size_t *size,
                        const ptrdiff_t *const strides[NOPS], void *const ptr[NOPS],
                        int key, bool reorder)
{
   if (ndims < 0 || ndims > OCH_MAX_DIMS) return set_error("invalid number of dimensions (%d)", ndims);
   s.nelem = 1; s.ndims = 0;
   for (int k = 0; k < NOPS; k++) s.ptr[k] = (char *)ptr[k];
   for (int d = 0; d < ndims; d++) s.nelem *= size[d];
   if (s.nelem == 0) return 0;
   for (int d = 0; d < ndims; d++)
   {  if (size[d] == 1) continue;
      int j = s.ndims++;
      s.size[j] = size[d];
      for (int k = 0; k < NOPS; k++) s.stride[k][j] = strides[k][d];
      if (reorder && s.stride[key][j] < 0)
      {  for (int k = 0; k < NOPS; k++)
         {  s.ptr[k] += s.stride[k][j] * (int64_t)(size[d] - 1);
            s.stride[k][j] = -s.stride[k][j];
         }
      }
   }
   if (reorder)
   {  for (int i = 1; i < s.ndims; i++)          /* insertion sort, ascending key strides */
      {  for (int j = i; j > 0; j--)
         {  bool swap = false;
            if (s.stride[key][j - 1] > s.stride[key][j]) swap = true;
            else if (s.stride[key][j - 1] == s.stride[key][j])
            {  for (int k = 0; k < NOPS; k++)
               {  if (s.stride[k][j - 1] == s.stride[k][j]) continue;
                  swap = s.stride[k][j - 1] > s.stride[k][j]; break;
               }
            }
            if (!swap) break;
            uint64_t t = s.size[j]; s.size[j] = s.size[j - 1]; s.size[j - 1] = t;
            for (int k = 0; k < NOPS; k++)
            {  int64_t r = s.stride[k][j]; s.stride[k][j] = s.stride[k][j - 1]; s.stride[k][j - 1] = r; }
         }
      }
   }
   if (s.ndims > 1)
   {  int j = 0;
      for (int i = 1; i < s.ndims; i++)
      {  bool merge = true;
         for (int k = 0; k < NOPS; k++)
            if (s.stride[k][i] != s.stride[k][j] * (int64_t)s.size[j]) { merge = false; break; }
         if (merge) s.size[j] *= s.size[i];
         else
         {  j++; s.size[j] = s.size[i];
            for (int k = 0; k < NOPS; k++) s.stride[k][j] = s.stride[k][i];
         }
      }
      s.ndims = j + 1;
   }
   if (s.ndims == 0)
   {  s.ndims = 1; s.size[0] = 1;
      for (int k = 0; k < NOPS; k++) s.stride[k][0] = 0;
   }
   return 0;
}

/* Elements one launch of the elementwise engine handles: 0xFFFF0000 (keeps block base + thread offset from wrapping in
   32 bits) unless och_elemwise_set_launch_limit has lowered it so that small tensors take the cutting path below. The
   reference switches its kernels to 64-bit indices instead (solid/src/core/gpu/op/apply_elemwise.c:66-99). */
uint64_t ew_launch_limit();

/* Launcher signature: (shape with every size < 2^32 and nelem < 2^32, vec flag, first flat index). A shape above the
   limit is cut along its outermost dimension into runs that fit (or walked index by index and cut further inside when
   one index of it is still too much); a one-dimensional shape into runs of a multiple of 64 elements, so that every
   run starts as aligned as the whole. The runs are launched one after the other on the caller's stream. */
template <int NOPS, class L>
static int ew_launch_chunked(EwShape<NOPS> s, uint64_t flat0, L &&launch)
{
   const uint64_t LIMIT = ew_launch_limit();
   if (s.nelem == 0) return 0;
   if (s.nelem <= LIMIT) return launch(s, flat0);
   int last = s.ndims - 1;
   uint64_t inner = s.nelem / s.size[last];
   const uint64_t run1 = (LIMIT >= (1ull << 30)) ? (1ull << 30) : ((LIMIT & ~63ull) ? (LIMIT & ~63ull) : 64);
   uint64_t chunk = (s.ndims == 1) ? run1 : (inner <= LIMIT ? LIMIT / inner : 0);
   if (chunk >= 1)
   {  for (uint64_t start = 0; start < s.size[last]; start += chunk)
      {  EwShape<NOPS> c = s;
         c.size[last] = (s.size[last] - start < chunk) ? (s.size[last] - start) : chunk;
         c.nelem = inner * c.size[last];
         for (int k = 0; k < NOPS; k++) c.ptr[k] = s.ptr[k] + (int64_t)start * s.stride[k][last];
         if (launch(c, flat0 + start * inner) != 0) return -1;
      }
      return 0;
   }
   for (uint64_t i = 0; i < s.size[last]; i++)
   {  EwShape<NOPS> c = s;
      c.ndims = last; c.nelem = inner;
      for (int k = 0; k < NOPS; k++) c.ptr[k] = s.ptr[k] + (int64_t)i * s.stride[k][last];
      if (ew_launch_chunked<NOPS>(c, flat0 + i * inner, launch) != 0) return -1;
   }
   return 0;
}

/* Fill kernel parameters for a VEC-wide launch; returns false when VEC does not fit */
/* even_inputs: the first `even_inputs` operands are inputs whose kernel can read a step-2 first dimension with wide
   loads (vecmode 2, see load_even) */
template <int NOPS>
static bool ew_params(EwParams<NOPS> &p, const EwShape<NOPS> &s, int vec, const int elemsize[NOPS], uint64_t flat0, int even_inputs = 0)
{
   if (s.size[0] % vec != 0) return false;
   p.ndims = s.ndims;
   p.unr = 1; p.block = OCH_EW_BLOCK;
   p.ngroups = (uint32_t)(s.nelem / vec);
   p.group0 = flat0;
   {  uint64_t bytes = 0;
      for (int k = 0; k < NOPS; k++) bytes += s.nelem * (uint64_t)elemsize[k];
      p.nt = (bytes >= OCH_EW_STREAM_BYTES) ? 1 : 0;
   }
   p.div[0] = make_fastdiv((uint32_t)(s.size[0] / vec));
   for (int d = 1; d < s.ndims; d++) p.div[d] = make_fastdiv((uint32_t)s.size[d]);
   for (int k = 0; k < NOPS; k++)
   {  p.ptr[k] = s.ptr[k];
      p.estride[k] = s.stride[k][0];
      p.gstride[k] = s.stride[k][0] * vec;
      for (int d = 0; d < OCH_MAX_DIMS; d++) p.stride[k][d] = (d < s.ndims) ? s.stride[k][d] : 0;
      int width = elemsize[k] * vec; if (width > 16) width = 16;
      bool v = (s.stride[k][0] == elemsize[k]) && (((uintptr_t)s.ptr[k]) % width == 0);
      for (int d = 1; d < s.ndims && v; d++) if (s.stride[k][d] % width != 0) v = false;
      p.vecmode[k] = v ? 1 : 0;
      if (!v && k < even_inputs && vec > 1 && elemsize[k] <= 4 && s.stride[k][0] == 2 * elemsize[k])
      {  int span = 2 * elemsize[k] * vec; if (span > 16) span = 16;
         bool e = (((uintptr_t)s.ptr[k]) % span == 0);
         for (int d = 1; d < s.ndims && e; d++) if (s.stride[k][d] % span != 0) e = false;
         if (e) p.vecmode[k] = 2;
      }
   }
   return true;
}

/* Parameters of the row kernels, or false when they do not apply: the destination (last operand) must have unit stride
   along dimension 0 and rows of at least 24 bytes, every operand must be aligned to its element, and the units of all
   rows must be countable in 32 bits. */
template <int NOPS>
static bool ew_rows_params(EwParams<NOPS> &p, const EwShape<NOPS> &s, int vec, const int elemsize[NOPS], uint64_t flat0)
{
   const int out = NOPS - 1;
   if (vec <= 1 || s.nelem == 0 || s.stride[out][0] != elemsize[out]) return false;
   const uint64_t n0 = s.size[0];
   if (n0 * elemsize[out] < 24) return false;
   for (int k = 0; k < NOPS; k++)
   {  if (((uintptr_t)s.ptr[k]) % elemsize[k] != 0) return false;
      for (int d = 0; d < s.ndims; d++) if (s.stride[k][d] % elemsize[k] != 0) return false;
   }
   const uint64_t chunks = row_units(n0, elemsize[out], vec);
   const uint64_t rows = s.nelem / n0;
   if (chunks > 0xFFFFFFFFull || rows * chunks > 0xFFFF0000ull) return false;
   p.ndims = s.ndims;
   p.unr = 1; p.block = OCH_EW_BLOCK;
   p.ngroups = (uint32_t)(rows * chunks);
   p.group0 = flat0;
   p.row_n0 = n0;
   {  uint64_t bytes = 0;
      for (int k = 0; k < NOPS; k++) bytes += s.nelem * (uint64_t)elemsize[k];
      p.nt = (bytes >= OCH_EW_STREAM_BYTES) ? 1 : 0;
   }
   p.div[0] = make_fastdiv((uint32_t)chunks);
   for (int d = 1; d < s.ndims; d++) p.div[d] = make_fastdiv((uint32_t)s.size[d]);
   for (int k = 0; k < NOPS; k++)
   {  p.ptr[k] = s.ptr[k];
      p.estride[k] = s.stride[k][0];
      p.gstride[k] = s.stride[k][0] * vec;
      for (int d = 0; d < OCH_MAX_DIMS; d++) p.stride[k][d] = (d < s.ndims) ? s.stride[k][d] : 0;
      p.vecmode[k] = (s.stride[k][0] == elemsize[k]) ? 1 : 0;
   }
   return true;
}

template <int NOPS>
static bool ew_rows_wanted(const EwShape<NOPS> &s, int vec, const int elemsize[NOPS])
{
   if (vec <= 1) return false;
   bool misfit = (s.ndims > 1 && s.size[0] % vec != 0);
   for (int k = 0; k < NOPS; k++)
   {  if (s.stride[k][0] != elemsize[k]) continue;
      int width = elemsize[k] * vec; if (width > 16) width = 16;
      if (((uintptr_t)s.ptr[k]) % width != 0) misfit = true;
      for (int d = 1; d < s.ndims; d++) if (s.stride[k][d] % width != 0) misfit = true;
   }
   return misfit;
}

template <class T> constexpr int vec_for() { return (16 / (int)sizeof(T)) > 0 ? (16 / (int)sizeof(T)) : 1; }
template <class A, class B, class C> constexpr int vec_for3()
{  constexpr int m = sizeof(A) > sizeof(B) ? (sizeof(A) > sizeof(C) ? sizeof(A) : sizeof(C)) : (sizeof(B) > sizeof(C) ? sizeof(B) : sizeof(C));
   return (16 / m) > 0 ? (16 / m) : 1;
}

#define OCH_EW_UNR 1

/* ---- generic launchers ------------------------------------------------------ */
/* Picks the kernel variant for one (chunk of a) normalised shape:
     wide  : every operand has aligned unit stride along dim 0 -> VEC-wide accesses only
     mixed : dim 0 divisible by VEC, some operands strided or broadcast
     single: one element per thread (odd sizes); for 1-D shapes only the tail uses it   */
/* Launcher signature: (parameters, workgroups, threads per workgroup) */
template <int NOPS, class LW, class LM, class LS, class LR>
static int ew_dispatch(const EwShape<NOPS> &s, uint64_t flat0, int vec, const int (&es)[NOPS],
                       LW &&wide, LM &&mixed, LS &&single, LR &&rows, bool streaming_form = true)
{
   /* streaming_form = false: a launch that only writes keeps the plain stores and the 256-thread workgroups whatever
      its size (a float32 fill of 268 MB: 6.0 TB/s in the streaming form, the write ceiling of 6.6 - 6.8 is reached
      by plain stores) */
   EwParams<NOPS> p;
   /* unit-stride rows that are not whole aligned vectors (see the row kernels): a width that VEC does not divide (a
      one-dimensional shape of such a length is cut into body and tail below instead), or a unit-stride operand whose
      start or pitch is not a multiple of its vector width */
   {  if (ew_rows_wanted<NOPS>(s, vec, es) && ew_rows_params<NOPS>(p, s, vec, es, flat0))
      {  rows(p, (p.ngroups + OCH_EW_BLOCK - 1) / OCH_EW_BLOCK, (uint32_t)OCH_EW_BLOCK);
         OCH_CHECK_LAUNCH();
         return 0;
      }
   }
   auto run = [&](const EwShape<NOPS> &sh, uint64_t f0) -> bool
   {  if (!ew_params<NOPS>(p, sh, vec, es, f0, NOPS - 1)) return false;      /* vec = 1 (16-byte elements) always fits */
      if (!streaming_form) p.nt = 0;
      bool all = true;
      for (int k = 0; k < NOPS; k++) all = all && (p.vecmode[k] == 1);
      const uint32_t block = p.nt ? OCH_EW_BLOCK_STREAM : OCH_EW_BLOCK;
      p.block = block;
      if (all) wide(p, (p.ngroups + block * OCH_EW_UNR - 1) / (block * OCH_EW_UNR), block);
      else
      {  /* operands with element accesses want two groups in flight per thread; when every operand is read or written
            in wide accesses (or is a broadcast) one group per thread and the larger workgroup stream faster */
         bool elementwise = false;
         for (int k = 0; k < NOPS; k++) if (p.vecmode[k] == 0 && p.estride[k] != 0) elementwise = true;
         if (elementwise) { p.unr = 2; p.block = OCH_EW_BLOCK; mixed(p, (p.ngroups + OCH_EW_BLOCK * 2 - 1) / (OCH_EW_BLOCK * 2), (uint32_t)OCH_EW_BLOCK); }
         else             { p.unr = 1; mixed(p, (p.ngroups + block - 1) / block, block); }
      }
      return true;
   };
   if (!run(s, flat0))
   {  if (vec > 1 && s.ndims == 1 && s.size[0] > (uint64_t)vec)
      {  EwShape<NOPS> body = s, tail = s;
         body.size[0] = s.size[0] - s.size[0] % vec; body.nelem = body.size[0];
         tail.size[0] = s.size[0] % vec; tail.nelem = tail.size[0];
         for (int k = 0; k < NOPS; k++) tail.ptr[k] = s.ptr[k] + (int64_t)body.size[0] * s.stride[k][0];
         run(body, flat0);
         ew_params<NOPS>(p, tail, 1, es, flat0 + body.nelem);
         single(p, 1u, (uint32_t)OCH_EW_BLOCK);
      }
      else
      {  ew_params<NOPS>(p, s, 1, es, flat0);
         single(p, (p.ngroups + OCH_EW_BLOCK - 1) / OCH_EW_BLOCK, (uint32_t)OCH_EW_BLOCK);
      }
   }
   OCH_CHECK_LAUNCH();
   return 0;
}


/* Decide whether a normalised shape should run on the tiled kernels and fill their parameters.
   The output (last operand) must have unit stride along dimension 0; the inputs that are
   contiguous along one other dimension d1 (and strided along dimension 0) go through LDS. */
template <int NOPS>
static bool ew_tile_params(TileParams<NOPS> &t, const EwShape<NOPS> &s, const int (&es)[NOPS], int tile, int vec,
                           dim3 &grid, size_t &lds_bytes, const int (&tilebytes)[NOPS])
{
   const int out = NOPS - 1;
   if (s.ndims < 2 || s.stride[out][0] != es[out]) return false;
   if (s.size[0] % vec != 0 || s.size[0] < 16) return false;
   auto is_trans = [&](int k, int d)
   {  return s.stride[k][d] == es[k] && s.stride[k][0] != es[k] && s.stride[k][0] != 0; };
   int d1 = -1;
   for (int d = 1; d < s.ndims && d1 < 0; d++)
      for (int k = 0; k < out; k++) if (is_trans(k, d)) { d1 = d; break; }
   if (d1 < 0 || s.size[d1] < 16) return false;
   for (int k = 0; k < NOPS; k++)            /* in-tile offsets are computed with 24-bit multiplies (tile_offset) */
   {  const int64_t lim = (int64_t)1 << 23;
      if (s.stride[k][0] >= lim || s.stride[k][0] <= -lim || s.stride[k][d1] >= lim || s.stride[k][d1] <= -lim) return false;
   }
   memset(&t, 0, sizeof(t));
   bool any = false; size_t lds = 0;
   for (int k = 0; k < NOPS; k++)
   {  t.ptr[k] = s.ptr[k]; t.s0[k] = s.stride[k][0]; t.s1[k] = s.stride[k][d1];
      bool tr = (k != out) && is_trans(k, d1);
      if (tr)
      {  int vk = 16 / es[k]; if (vk < 1) vk = 1;
         if (s.size[d1] % vk != 0 || ((uintptr_t)s.ptr[k]) % 16 != 0) tr = false;
         for (int d = 0; d < s.ndims && tr; d++) if (d != d1 && s.stride[k][d] % 16 != 0) tr = false;
      }
      t.trans[k] = tr ? 1 : 0;
      if (tr) { any = true; t.lds_off[k] = (int)lds; lds += tilebytes[k]; }
      int width = es[k] * vec; if (width > 16) width = 16;
      bool v = (s.stride[k][0] == es[k]) && (((uintptr_t)s.ptr[k]) % width == 0);
      for (int d = 1; d < s.ndims && v; d++) if (s.stride[k][d] % width != 0) v = false;
      t.vecmode[k] = v ? 1 : 0;
   }
   if (!any || lds > 64 * 1024) return false;
   uint64_t outer = 1; t.nouter = 0;
   for (int d = 1; d < s.ndims; d++)
   {  if (d == d1) continue;
      t.odiv[t.nouter] = make_fastdiv((uint32_t)s.size[d]);
      for (int k = 0; k < NOPS; k++) t.so[k][t.nouter] = s.stride[k][d];
      t.nouter++; outer *= s.size[d];
   }
   uint64_t tiles0 = (s.size[0] + tile - 1) / tile, tiles1 = (s.size[d1] + tile - 1) / tile;
   if (outer > 65535 || tiles1 > 65535 || s.size[0] >= 0x40000000ull || s.size[d1] >= 0x40000000ull) return false;
   t.rowdiv = make_fastdiv((uint32_t)tiles1);
   t.n0 = (uint32_t)s.size[0]; t.n1 = (uint32_t)s.size[d1];
   {  uint64_t bytes = 0;
      for (int k = 0; k < NOPS; k++) bytes += s.nelem * (uint64_t)es[k];
      t.nt = (bytes >= OCH_EW_STREAM_BYTES) ? 1 : 0;
      t.diagonal = 0;
      for (int k = 0; k < NOPS; k++)
      {  const uint64_t pitch = (uint64_t)(t.s0[k] < 0 ? -t.s0[k] : t.s0[k]);
         if (t.trans[k] && pitch >= 16384 && pitch <= 65536 && (pitch & (pitch - 1)) == 0) t.diagonal = 1;
      }
   }
   grid = dim3((unsigned)tiles0, (unsigned)tiles1, (unsigned)outer);
   lds_bytes = lds;
   return true;
}

template <class F>
static int launch_ew3(int ndims, const size_t *size,
                      const ptrdiff_t *st1, void *p1, const ptrdiff_t *st2, void *p2,
                      const ptrdiff_t *st3, void *p3, hipStream_t stream)
{
   typedef typename F::A A; typedef typename F::B B; typedef typename F::R R;
   constexpr int VEC = vec_for3<A, B, R>();
   const ptrdiff_t *strides[3] = { st1, st2, st3 }; void *ptrs[3] = { p1, p2, p3 };
   EwShape<3> shape;
   if (ew_normalize<3>(shape, ndims, size, strides, ptrs, 2, true) != 0) return -1;
   const int es[3] = { (int)sizeof(A), (int)sizeof(B), (int)sizeof(R) };
   return ew_launch_chunked<3>(shape, 0, [&](const EwShape<3> &s, uint64_t flat0) -> int
   {  constexpr size_t MAXS = sizeof(A) > sizeof(B) ? (sizeof(A) > sizeof(R) ? sizeof(A) : sizeof(R)) : (sizeof(B) > sizeof(R) ? sizeof(B) : sizeof(R));
      constexpr int TILE = tile_dim(MAXS);
      const int tb[3] = { tile_bytes<A>(TILE), tile_bytes<B>(TILE), 0 };
      TileParams<3> tp; dim3 grid; size_t lds;
      if (ew_tile_params<3>(tp, s, es, TILE, VEC, grid, lds, tb))
      {  if (tp.nt) hipLaunchKernelGGL((ew3_tile_kernel<F, VEC, true>), grid, dim3(tile_threads(MAXS)), lds, stream, tp);
         else       hipLaunchKernelGGL((ew3_tile_kernel<F, VEC, false>), grid, dim3(tile_threads(MAXS)), lds, stream, tp);
         OCH_CHECK_LAUNCH();
         return 0;
      }
      return ew_dispatch<3>(s, flat0, VEC, es,
         [&](const EwParams<3> &p, uint32_t blocks, uint32_t threads)
         {  if (p.nt) hipLaunchKernelGGL((ew3_kernel<F, VEC, OCH_EW_UNR, true, true>), dim3(blocks), dim3(threads), 0, stream, p);
            else      hipLaunchKernelGGL((ew3_kernel<F, VEC, OCH_EW_UNR, true, false>), dim3(blocks), dim3(threads), 0, stream, p); },
         [&](const EwParams<3> &p, uint32_t blocks, uint32_t threads)
         {  /* nontemporal accesses reach only the operands that take the wide path; a broadcast operand keeps its cached loads */
            if (p.nt) hipLaunchKernelGGL((ew3_kernel<F, VEC, 2, false, true>), dim3(blocks), dim3(threads), 0, stream, p);
            else      hipLaunchKernelGGL((ew3_kernel<F, VEC, 2, false, false>), dim3(blocks), dim3(threads), 0, stream, p); },
         [&](const EwParams<3> &p, uint32_t blocks, uint32_t threads)
         {  hipLaunchKernelGGL((ew3_kernel<F, 1, 1, false>), dim3(blocks), dim3(threads), 0, stream, p); },
         [&](const EwParams<3> &p, uint32_t blocks, uint32_t threads)
         {  if constexpr (VEC > 1)
            {  if (p.nt) hipLaunchKernelGGL((ew3_rows_kernel<F, VEC, true>), dim3(blocks), dim3(threads), 0, stream, p);
               else      hipLaunchKernelGGL((ew3_rows_kernel<F, VEC, false>), dim3(blocks), dim3(threads), 0, stream, p);
            } });
   });
}

template <class F>
static int launch_ew2(int ndims, const size_t *size,
                      const ptrdiff_t *st1, void *p1, const ptrdiff_t *st2, void *p2, hipStream_t stream)
{
   typedef typename F::A A; typedef typename F::R R;
   constexpr int VEC = vec_for3<A, A, R>();
   const ptrdiff_t *strides[2] = { st1, st2 }; void *ptrs[2] = { p1, p2 };
   EwShape<2> shape;
   if (ew_normalize<2>(shape, ndims, size, strides, ptrs, 1, true) != 0) return -1;
   const int es[2] = { (int)sizeof(A), (int)sizeof(R) };
   return ew_launch_chunked<2>(shape, 0, [&](const EwShape<2> &s, uint64_t flat0) -> int
   {  constexpr size_t MAXS = sizeof(A) > sizeof(R) ? sizeof(A) : sizeof(R);
      constexpr int TILE = tile_dim(MAXS);
      const int tb[2] = { tile_bytes<A>(TILE), 0 };
      TileParams<2> tp; dim3 grid; size_t lds;
      if (ew_tile_params<2>(tp, s, es, TILE, VEC, grid, lds, tb))
      {  if (tp.nt) hipLaunchKernelGGL((ew2_tile_kernel<F, VEC, true>), grid, dim3(tile_threads(MAXS)), lds, stream, tp);
         else       hipLaunchKernelGGL((ew2_tile_kernel<F, VEC, false>), grid, dim3(tile_threads(MAXS)), lds, stream, tp);
         OCH_CHECK_LAUNCH();
         return 0;
      }
      return ew_dispatch<2>(s, flat0, VEC, es,
         [&](const EwParams<2> &p, uint32_t blocks, uint32_t threads)
         {  if (p.nt) hipLaunchKernelGGL((ew2_kernel<F, VEC, OCH_EW_UNR, true, true>), dim3(blocks), dim3(threads), 0, stream, p);
            else      hipLaunchKernelGGL((ew2_kernel<F, VEC, OCH_EW_UNR, true, false>), dim3(blocks), dim3(threads), 0, stream, p); },
         [&](const EwParams<2> &p, uint32_t blocks, uint32_t threads)
         {  if (p.nt) hipLaunchKernelGGL((ew2_kernel<F, VEC, 2, false, true>), dim3(blocks), dim3(threads), 0, stream, p);
            else      hipLaunchKernelGGL((ew2_kernel<F, VEC, 2, false, false>), dim3(blocks), dim3(threads), 0, stream, p); },
         [&](const EwParams<2> &p, uint32_t blocks, uint32_t threads)
         {  hipLaunchKernelGGL((ew2_kernel<F, 1, 1, false>), dim3(blocks), dim3(threads), 0, stream, p); },
         [&](const EwParams<2> &p, uint32_t blocks, uint32_t threads)
         {  if constexpr (VEC > 1)
            {  if (p.nt) hipLaunchKernelGGL((ew2_rows_kernel<F, VEC, true>), dim3(blocks), dim3(threads), 0, stream, p);
               else      hipLaunchKernelGGL((ew2_rows_kernel<F, VEC, false>), dim3(blocks), dim3(threads), 0, stream, p);
            } });
   });
}

/* reorder=false for functors that use the flat index */
template <class F>
static int launch_ew1(int ndims, const size_t *size, const ptrdiff_t *st, void *ptr,
                      const typename F::Param &prm, bool reorder, hipStream_t stream)
{
   typedef typename F::R R;
   constexpr int VEC = vec_for<R>();
   const ptrdiff_t *strides[1] = { st }; void *ptrs[1] = { ptr };
   EwShape<1> shape;
   if (ew_normalize<1>(shape, ndims, size, strides, ptrs, 0, reorder) != 0) return -1;
   const int es[1] = { (int)sizeof(R) };
   return ew_launch_chunked<1>(shape, 0, [&](const EwShape<1> &s, uint64_t flat0) -> int
   {  return ew_dispatch<1>(s, flat0, VEC, es,
         [&](const EwParams<1> &p, uint32_t blocks, uint32_t threads)
         {  if (p.nt) hipLaunchKernelGGL((ew1_kernel<F, VEC, OCH_EW_UNR, true, true>), dim3(blocks), dim3(threads), 0, stream, p, prm);
            else      hipLaunchKernelGGL((ew1_kernel<F, VEC, OCH_EW_UNR, true, false>), dim3(blocks), dim3(threads), 0, stream, p, prm); },
         [&](const EwParams<1> &p, uint32_t blocks, uint32_t threads)
         {  hipLaunchKernelGGL((ew1_kernel<F, VEC, 2, false>), dim3(blocks), dim3(threads), 0, stream, p, prm); },
         [&](const EwParams<1> &p, uint32_t blocks, uint32_t threads)
         {  hipLaunchKernelGGL((ew1_kernel<F, 1, 1, false>), dim3(blocks), dim3(threads), 0, stream, p, prm); },
         [&](const EwParams<1> &p, uint32_t blocks, uint32_t threads)
         {  if constexpr (VEC > 1)
            {  if (p.nt) hipLaunchKernelGGL((ew1_rows_kernel<F, VEC, true>), dim3(blocks), dim3(threads), 0, stream, p, prm);
               else      hipLaunchKernelGGL((ew1_rows_kernel<F, VEC, false>), dim3(blocks), dim3(threads), 0, stream, p, prm);
            } }, F::RMW);
   });
}

} /* namespace och */
