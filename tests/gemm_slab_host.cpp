/* Host walk through the LDS layout of the pipelined float and double GEMM (csrc/och_gemm_f32p_slab.h, och_gemm_f64p_slab.h), for
   tests/test_gemm_layout_cpu.py. For every operand layout (contiguous along k or along the rows) and every block tile
   (256, 128, 64 rows) a slab of a synthetic matrix is brought into an LDS image by exactly the offsets the kernel's load
   instructions use (4 waves x LOADS instructions x 64 lanes x 16 bytes), and every value an MFMA would get -- tile i of a
   wave, step t of quad q, lane l -- is compared with the matrix element it has to be: row wbase + row(i, l % 32),
   k = 8 q + 4 (l / 32) + t. Also checked: loads stay inside the slab of the rows that exist, no two loads write the same
   LDS bytes, everything lies inside the operand's LDS area. Returns the number of violations. */
#include <stdint.h>
#include <string.h>
#include <stdio.h>
#include <vector>
#include "och_gemm_f32p_slab.h"
#include "och_gemm_f64p_slab.h"
#include "och_gemm_c32p_slab.h"
#include "och_gemm_c64p_slab.h"

using namespace och;

template <bool KC, int ROWS>
static long check(uint32_t rows /* rows of the tile that exist: a multiple of 4 */, int64_t ld, int verbose)
{
   typedef FloatSlab<KC, ROWS> L;
   constexpr int KT = 32, TS = L::TS;
   long bad = 0;
   /* the matrix around the slab: element (row r, k) = 1000 r + k + 1, stored as the kernel's operand layout says */
   const int64_t nrow = ROWS, nk = KT;
   std::vector<float> mat((size_t)(KC ? nrow * ld : nk * ld), -1.0f);
   auto element = [&](int64_t r, int64_t k) -> float & { return mat[(size_t)(KC ? r * ld + k : k * ld + r)]; };
   for (int64_t r = 0; r < (int64_t)rows; r++) for (int64_t k = 0; k < nk; k++) element(r, k) = (float)(1000 * r + k + 1);
   const char *base = L::slab_base(reinterpret_cast<const char *>(mat.data()), ld, 0, 0);
   std::vector<char> lds(L::OPERAND, 0);
   std::vector<unsigned char> written(L::OPERAND, 0);
   for (uint32_t wave = 0; wave < 4; wave++)
      for (int j = 0; j < L::LOADS; j++)
         for (uint32_t lane = 0; lane < 64; lane++)
         {  const uint32_t off = L::load_offset(j, wave, lane, ld, rows), tgt = L::load_target(j, wave) + 16 * lane;
            if (tgt % 16 != 0 || tgt + 16 > (uint32_t)L::OPERAND) { bad++; continue; }
            if ((size_t)off + 16 > mat.size() * 4) { bad++; continue; }
            float v[4]; memcpy(v, base + off, 16);
            for (int e = 0; e < 4; e++) if (v[e] < 0) bad++;                  /* a load outside the rows that exist */
            for (int e = 0; e < 16; e++) { if (written[tgt + e]) bad++; written[tgt + e] = 1; }
            memcpy(lds.data() + tgt, base + off, 16);
         }
   /* rows past the end of the matrix hold the last rows that exist (the kernel never writes their results) */
   auto expected = [&](uint32_t r, uint32_t k) -> float
   {  uint32_t src = r;
      if (r >= rows) src = KC ? rows - 1 : rows - 4 + r % 4;
      return (float)(1000 * src + k + 1);
   };
   const int wave_rows = 32 * TS;
   for (uint32_t wbase = 0; wbase < (uint32_t)ROWS; wbase += wave_rows)
      for (uint32_t lane = 0; lane < 64; lane++)
         for (int q = 0; q < 4; q++)
         {  och_f32x4 f[4];
            for (int x = 0; x < 4; x++) f[x] = och_f32x4{0, 0, 0, 0};
            for (int x = 0; x < L::READS; x++)
            {  const uint32_t at = L::read_lane(wbase, lane) + L::read_offset(x, q);
               const uint32_t width = (KC || TS == 4) ? 16 : 4 * TS;                  /* bytes of the fragment read */
               if (at % width != 0 || at + width > (uint32_t)L::OPERAND) { bad++; continue; }
               f[x] = L::read(lds.data() + at);
            }
            for (int i = 0; i < TS; i++)
               for (int t = 0; t < 4; t++)
               {  const uint32_t r = wbase + L::row(i, lane % 32), k = 8 * q + 4 * (lane / 32) + t;
                  const float got = L::value(f, i, t), want = expected(r, k);
                  if (got != want)
                  {  if (verbose && bad < 10) printf("KC=%d ROWS=%d rows=%u: tile %d step %d quad %d lane %u: got %g, want %g\n", (int)KC, ROWS, rows, i, t, q, lane, got, want);
                     bad++;
                  }
               }
         }
   return bad;
}

extern "C" long gemm_slab_check(int kc, int rows_of_tile, unsigned rows, long ld, int verbose)
{
   if (kc) { if (rows_of_tile == 256) return check<true, 256>(rows, ld, verbose); if (rows_of_tile == 128) return check<true, 128>(rows, ld, verbose); if (rows_of_tile == 64) return check<true, 64>(rows, ld, verbose); }
   else    { if (rows_of_tile == 256) return check<false, 256>(rows, ld, verbose); if (rows_of_tile == 128) return check<false, 128>(rows, ld, verbose); if (rows_of_tile == 64) return check<false, 64>(rows, ld, verbose); }
   return -1;
}

/* The double kernel: slabs of 16 k, a wave owns half the rows of its operand as TILES tiles of 16 rows; v_mfma_f64_16x16x4
   takes one double per lane and operand, lanes 16 g .. 16 g + 15 holding k-group g: in step t of pair P, k = 8 P + 2 g + t. */
template <bool KC, int ROWS>
static long check_double(uint32_t rows /* a multiple of 2 */, int64_t ld, int verbose)
{
   typedef DoubleSlab<KC, ROWS> L;
   constexpr int KT = OCH_DP_KT, TILES = L::TILES, AREA = KC ? 8 * L::PLANE : 16 * L::ROWP;
   long bad = 0;
   std::vector<double> mat((size_t)(KC ? (int64_t)ROWS * ld : (int64_t)KT * ld), -1.0);
   auto element = [&](int64_t r, int64_t k) -> double & { return mat[(size_t)(KC ? r * ld + k : k * ld + r)]; };
   for (int64_t r = 0; r < (int64_t)rows; r++) for (int64_t k = 0; k < KT; k++) element(r, k) = (double)(1000 * r + k + 1);
   const char *base = L::slab_base(reinterpret_cast<const char *>(mat.data()), ld, 0, 0);
   std::vector<char> lds(AREA, 0);
   std::vector<unsigned char> written(AREA, 0);
   for (uint32_t wave = 0; wave < 4; wave++)
      for (int j = 0; j < L::LOADS; j++)
         for (uint32_t lane = 0; lane < 64; lane++)
         {  const uint32_t off = L::load_offset(j, wave, lane, ld, rows), tgt = L::load_target(j, wave) + 16 * lane;
            if (tgt % 16 != 0 || tgt + 16 > (uint32_t)AREA) { bad++; continue; }
            if ((size_t)off + 16 > mat.size() * 8) { bad++; continue; }
            double v[2]; memcpy(v, base + off, 16);
            for (int e = 0; e < 2; e++) if (v[e] < 0) bad++;
            for (int e = 0; e < 16; e++) { if (written[tgt + e]) bad++; written[tgt + e] = 1; }
            memcpy(lds.data() + tgt, base + off, 16);
         }
   auto expected = [&](uint32_t r, uint32_t k) -> double
   {  uint32_t src = r;
      if (r >= rows) src = KC ? rows - 1 : rows - 2 + r % 2;
      return (double)(1000 * src + k + 1);
   };
   for (uint32_t wbase = 0; wbase < (uint32_t)ROWS; wbase += ROWS / 2)
      for (uint32_t lane = 0; lane < 64; lane++)
         for (int P = 0; P < KT / 8; P++)
         {  och_f64x2 f[TILES];
            for (int x = 0; x < TILES; x++)
            {  f[x] = och_f64x2{0, 0};
               const uint32_t at = L::read_lane(wbase, lane) + L::read_offset(x, P);
               if (at % 16 != 0 || at + 16 > (uint32_t)AREA) { bad++; continue; }
               memcpy(&f[x], lds.data() + at, 16);
            }
            for (int i = 0; i < TILES; i++)
               for (int t = 0; t < 2; t++)
               {  const uint32_t r = wbase + L::row(i, lane % 16), k = 8 * P + 2 * (lane / 16) + t;
                  const double got = L::value(f, i, t), want = expected(r, k);
                  if (got != want)
                  {  if (verbose && bad < 10) printf("double KC=%d ROWS=%d rows=%u: tile %d step %d pair %d lane %u: got %g, want %g\n", (int)KC, ROWS, rows, i, t, P, lane, got, want);
                     bad++;
                  }
               }
         }
   return bad;
}

extern "C" long gemm_slab_check_double(int kc, int rows_of_tile, unsigned rows, long ld, int verbose)
{
   if (kc) { if (rows_of_tile == 256) return check_double<true, 256>(rows, ld, verbose); if (rows_of_tile == 128) return check_double<true, 128>(rows, ld, verbose); }
   else    { if (rows_of_tile == 256) return check_double<false, 256>(rows, ld, verbose); if (rows_of_tile == 128) return check_double<false, 128>(rows, ld, verbose); }
   return -1;
}

/* The complex kernels: element (r, k) = (v, -v - 0.5) with v = 1000 r + k + 1.
   complex float: slabs of 128 rows and 32 k, waves of 64 rows as two tiles of 32; in step t of quad q lane l holds
   k = 8 q + 4 (t / 2) + 2 (l / 32) + t % 2 (both operands use the same map, which is all the product needs; it covers the
   eight k of a quad once). complex double: slabs of 128 or 64 rows and 16 k, [k][row][re, im], waves of half the rows as
   tiles of 16; in step t of pair P lane l holds k = 8 P + 4 t + l / 16. */
template <bool KC>
static long check_cfloat(uint32_t rows /* a multiple of 2 */, int64_t ld, int verbose)
{
   typedef CFloatSlab<KC> L;
   constexpr int KT = 32, ROWS = 128, AREA = OCH_CP_OPERAND;
   long bad = 0;
   std::vector<float> mat((size_t)(KC ? (int64_t)ROWS * ld : (int64_t)KT * ld) * 2, 1.0f);      /* 1: never a valid part */
   auto at = [&](int64_t r, int64_t k) -> float * { return &mat[(size_t)(KC ? r * ld + k : k * ld + r) * 2]; };
   auto re = [](int64_t r, int64_t k) { return (float)(1000 * r + k + 2); };
   for (int64_t r = 0; r < (int64_t)rows; r++) for (int64_t k = 0; k < KT; k++) { at(r, k)[0] = re(r, k); at(r, k)[1] = -re(r, k) - 0.5f; }
   const char *base = L::slab_base(reinterpret_cast<const char *>(mat.data()), ld, 0, 0);
   std::vector<char> lds(AREA, 0);
   std::vector<unsigned char> written(AREA, 0);
   for (uint32_t wave = 0; wave < 4; wave++)
      for (int j = 0; j < 8; j++)
         for (uint32_t lane = 0; lane < 64; lane++)
         {  const uint32_t off = L::load_offset(j, wave, lane, ld, rows), tgt = L::load_target(j, wave) + 16 * lane;
            if (tgt % 16 != 0 || tgt + 16 > (uint32_t)AREA || (size_t)off + 16 > mat.size() * 4) { bad++; continue; }
            float v[4]; memcpy(v, base + off, 16);
            for (int e = 0; e < 4; e++) if (v[e] == 1.0f) bad++;
            for (int e = 0; e < 16; e++) { if (written[tgt + e]) bad++; written[tgt + e] = 1; }
            memcpy(lds.data() + tgt, base + off, 16);
         }
   auto expected = [&](uint32_t r, uint32_t k, int c) -> float
   {  uint32_t src = r;
      if (r >= rows) src = KC ? rows - 1 : rows - 2 + r % 2;
      return c == 0 ? re(src, k) : -re(src, k) - 0.5f;
   };
   for (uint32_t wbase = 0; wbase < (uint32_t)ROWS; wbase += 64)
      for (uint32_t lane = 0; lane < 64; lane++)
         for (int q = 0; q < 4; q++)
         {  och_f32x4 f[4];
            for (int x = 0; x < 4; x++)
            {  f[x] = och_f32x4{0, 0, 0, 0};
               const uint32_t a = L::read_lane(wbase, lane) + L::read_offset(x, q);
               if (a % 16 != 0 || a + 16 > (uint32_t)AREA) { bad++; continue; }
               memcpy(&f[x], lds.data() + a, 16);
            }
            for (int i = 0; i < 2; i++) for (int t = 0; t < 4; t++) for (int c = 0; c < 2; c++)
            {  const uint32_t r = wbase + L::row(i, lane % 32), k = 8 * q + 4 * (t / 2) + 2 * (lane / 32) + t % 2;
               const float got = L::value(f, i, t, c), want = expected(r, k, c);
               if (got != want)
               {  if (verbose && bad < 10) printf("cfloat KC=%d rows=%u: tile %d step %d part %d quad %d lane %u: got %g, want %g\n", (int)KC, rows, i, t, c, q, lane, got, want);
                  bad++;
               }
            }
         }
   return bad;
}

template <bool KC, int ROWS>
static long check_cdouble(uint32_t rows, int64_t ld, int verbose)
{
   typedef CDoubleSlab<KC, ROWS> L;
   constexpr int KT = OCH_ZP_KT, TILES = L::TILES, AREA = 16 * L::PLANE;
   long bad = 0;
   std::vector<double> mat((size_t)(KC ? (int64_t)ROWS * ld : (int64_t)KT * ld) * 2, 1.0);
   auto at = [&](int64_t r, int64_t k) -> double * { return &mat[(size_t)(KC ? r * ld + k : k * ld + r) * 2]; };
   auto re = [](int64_t r, int64_t k) { return (double)(1000 * r + k + 2); };
   for (int64_t r = 0; r < (int64_t)rows; r++) for (int64_t k = 0; k < KT; k++) { at(r, k)[0] = re(r, k); at(r, k)[1] = -re(r, k) - 0.5; }
   const char *base = L::slab_base(reinterpret_cast<const char *>(mat.data()), ld, 0, 0);
   std::vector<char> lds(AREA, 0);
   std::vector<unsigned char> written(AREA, 0);
   for (uint32_t wave = 0; wave < 4; wave++)
      for (int j = 0; j < L::LOADS; j++)
         for (uint32_t lane = 0; lane < 64; lane++)
         {  const uint32_t off = L::load_offset(j, wave, lane, ld, rows), tgt = L::load_target(j, wave) + 16 * lane;
            if (tgt % 16 != 0 || tgt + 16 > (uint32_t)AREA || (size_t)off + 16 > mat.size() * 8) { bad++; continue; }
            double v[2]; memcpy(v, base + off, 16);
            for (int e = 0; e < 2; e++) if (v[e] == 1.0) bad++;
            for (int e = 0; e < 16; e++) { if (written[tgt + e]) bad++; written[tgt + e] = 1; }
            memcpy(lds.data() + tgt, base + off, 16);
         }
   auto expected = [&](uint32_t r, uint32_t k, int c) -> double
   {  const uint32_t src = r >= rows ? rows - 1 : r;
      return c == 0 ? re(src, k) : -re(src, k) - 0.5;
   };
   for (uint32_t wbase = 0; wbase < (uint32_t)ROWS; wbase += ROWS / 2)
      for (uint32_t lane = 0; lane < 64; lane++)
         for (int P = 0; P < KT / 8; P++)
         {  och_f64x2 f[L::READS];
            for (int x = 0; x < L::READS; x++)
            {  f[x] = och_f64x2{0, 0};
               const uint32_t a = L::read_lane(wbase, lane) + L::read_offset(x, P);
               if (a % 16 != 0 || a + 16 > (uint32_t)AREA) { bad++; continue; }
               memcpy(&f[x], lds.data() + a, 16);
            }
            for (int i = 0; i < TILES; i++) for (int t = 0; t < 2; t++) for (int c = 0; c < 2; c++)
            {  const uint32_t r = wbase + L::row(i, lane % 16), k = 8 * P + 4 * t + lane / 16;
               const double got = L::value(f, i, t, c), want = expected(r, k, c);
               if (got != want)
               {  if (verbose && bad < 10) printf("cdouble KC=%d ROWS=%d rows=%u: tile %d step %d part %d pair %d lane %u: got %g, want %g\n", (int)KC, ROWS, rows, i, t, c, P, lane, got, want);
                  bad++;
               }
            }
         }
   return bad;
}

extern "C" long gemm_slab_check_cfloat(int kc, unsigned rows, long ld, int verbose)
{  return kc ? check_cfloat<true>(rows, ld, verbose) : check_cfloat<false>(rows, ld, verbose); }
extern "C" long gemm_slab_check_cdouble(int kc, int rows_of_tile, unsigned rows, long ld, int verbose)
{
   if (kc) { if (rows_of_tile == 128) return check_cdouble<true, 128>(rows, ld, verbose); if (rows_of_tile == 64) return check_cdouble<true, 64>(rows, ld, verbose); }
   else    { if (rows_of_tile == 128) return check_cdouble<false, 128>(rows, ld, verbose); if (rows_of_tile == 64) return check_cdouble<false, 64>(rows, ld, verbose); }
   return -1;
}
