/* TEST INFRASTRUCTURE (see oracle_types.h).
 * Includes the file named by O_TMPL_FILE once for each of the 15 element types with
 *   TN type name, T C type, UT unsigned twin (integers), PN real-part type name,
 *   WN / W work type name and C type, MF(fn) math function of W precision,
 *   K_BOOL / K_UINT / K_SINT / K_FLOAT / K_COMPLEX kind flags (exactly one is 1),
 *   HALF_OR_INF the CPU function table's infinity constant of the part type (complex).
 */
#ifndef O_TMPL_FILE
#error "O_TMPL_FILE must name the per-type template"
#endif
#define K_BOOL 1
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN bool
#define T o_bool
#define PN bool
#define WN bool
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 1
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN uint8
#define T uint8_t
#define PN uint8
#define WN uint8
#define UT uint8_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 1
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN uint16
#define T uint16_t
#define PN uint16
#define WN uint16
#define UT uint16_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 1
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN uint32
#define T uint32_t
#define PN uint32
#define WN uint32
#define UT uint32_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 1
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN uint64
#define T uint64_t
#define PN uint64
#define WN uint64
#define UT uint64_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 1
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN int8
#define T int8_t
#define PN int8
#define WN int8
#define UT uint8_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 1
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN int16
#define T int16_t
#define PN int16
#define WN int16
#define UT uint16_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 1
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN int32
#define T int32_t
#define PN int32
#define WN int32
#define UT uint32_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 1
#define K_FLOAT 0
#define K_COMPLEX 0
#define TN int64
#define T int64_t
#define PN int64
#define WN int64
#define UT uint64_t
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef UT
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 1
#define K_COMPLEX 0
#define TN half
#define T o_half
#define PN half
#define WN float
#define W float
#define MF(fn) fn##f
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef W
#undef MF
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 1
#define K_COMPLEX 0
#define TN float
#define T float
#define PN float
#define WN float
#define W float
#define MF(fn) fn##f
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef W
#undef MF
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 1
#define K_COMPLEX 0
#define TN double
#define T double
#define PN double
#define WN double
#define W double
#define MF(fn) fn
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef W
#undef MF
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 1
#define TN chalf
#define T o_chalf
#define PN half
#define WN float
#define W float
#define MF(fn) fn##f
#define HALF_OR_INF ((o_half)0xFC00)
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef W
#undef MF
#undef HALF_OR_INF
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 1
#define TN cfloat
#define T o_cfloat
#define PN float
#define WN float
#define W float
#define MF(fn) fn##f
#define HALF_OR_INF ((float)(1. / 0.))
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef W
#undef MF
#undef HALF_OR_INF
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

#define K_BOOL 0
#define K_UINT 0
#define K_SINT 0
#define K_FLOAT 0
#define K_COMPLEX 1
#define TN cdouble
#define T o_cdouble
#define PN double
#define WN double
#define W double
#define MF(fn) fn
#define HALF_OR_INF ((double)(1. / 0.))
#include O_TMPL_FILE
#undef TN
#undef T
#undef PN
#undef WN
#undef W
#undef MF
#undef HALF_OR_INF
#undef K_BOOL
#undef K_UINT
#undef K_SINT
#undef K_FLOAT
#undef K_COMPLEX

