/* Where the slabs of the pipelined double GEMM (och_gemm_f64p.hip) lie in LDS: which bytes a load instruction of a wave
   fetches and where it puts them, where a lane reads its fragments, and which row and k of the operand a fragment value
   is. Index arithmetic only, so that a host program can walk through it (tests/gemm_slab_host.cpp). */
#pragma once
#include <stdint.h>

#ifndef OCH_SLAB_FN
#  if defined(__HIPCC__)
#     define OCH_SLAB_FN __host__ __device__ __forceinline__
#  else
#     define OCH_SLAB_FN inline
#  endif
#endif

#define OCH_DP_KT 16

namespace och {

typedef double och_f64x2 __attribute__((ext_vector_type(2)));

/* one operand's slab of ROWS rows: where its loads come from and go to, where the fragments are read, which row a
   fragment value belongs to */
template <bool KC, int ROWS>
struct DoubleSlab
{
   static constexpr int PLANE = ROWS * 16 + 128;     /* KC: bytes per chunk plane */
   static constexpr int ROWP = ROWS * 8 + 64;        /* !KC: bytes per k */
   static constexpr int LOADS = ROWS * OCH_DP_KT * 8 / 1024 / 4;      /* loads per wave and slab: 8 or 4 */
   static constexpr int TILES = ROWS / 2 / 16;       /* tiles per wave: 8 or 4; also the fragment reads per pair */
   static constexpr int GROUPS = ROWS / 64, PARTS = ROWS / 128;
   /* load j of wave w. KC: chunk (w / GROUPS) * LOADS + j of the 64 rows of group w % GROUPS; !KC: unit u = w * LOADS + j
      is part u % PARTS (128 rows) of k = u / PARTS */
   /* `rows`: how many of the tile's rows exist (a multiple of 2; fewer than ROWS in the last tile of a matrix whose size is
      not a multiple of the tile). Lanes whose rows do not exist fetch the last rows that do: loads stay inside the matrix,
      and what they bring is multiplied into rows of the tile that are never written. */
   static OCH_SLAB_FN uint32_t load_offset(int j, uint32_t wave, uint32_t lane, int64_t ld, uint32_t rows)
   {  if (KC)
      {  uint32_t row = (wave % GROUPS) * 64 + lane;
         row = row < rows ? row : rows - 1;
         return (uint32_t)((int64_t)row * ld * 8 + ((wave / GROUPS) * LOADS + j) * 16);
      }
      const uint32_t u = wave * LOADS + j;
      uint32_t row = (u % PARTS) * 128 + lane * 2;
      row = row < rows ? row : rows - 2;
      return (uint32_t)((int64_t)(u / PARTS) * ld * 8 + row * 8);
   }
   static OCH_SLAB_FN uint32_t load_target(int j, uint32_t wave)
   {  if (KC) return ((wave / GROUPS) * LOADS + j) * PLANE + (wave % GROUPS) * 1024;
      const uint32_t u = wave * LOADS + j;
      return (u / PARTS) * ROWP + (u % PARTS) * 1024;
   }
   static OCH_SLAB_FN const char *slab_base(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0)
   {  return mat + (KC ? ((int64_t)k0 + (int64_t)mn0 * ld) : ((int64_t)mn0 + (int64_t)k0 * ld)) * 8; }
   /* fragment read x (0 .. TILES - 1) of pair P: the lane's part of the address, and the immediate part */
   static OCH_SLAB_FN uint32_t read_lane(uint32_t wbase, uint32_t lane)
   {  const uint32_t r = lane % 16, kg = lane / 16;
      return KC ? kg * PLANE + (wbase + r) * 16 : 2 * kg * ROWP + (wbase + 2 * r) * 8;
   }
   static constexpr uint32_t read_offset(int x, int P)
   {  return KC ? (uint32_t)(4 * P * PLANE + x * 256) : (uint32_t)((8 * P + x / (TILES / 2)) * ROWP + (x % (TILES / 2)) * 256); }
   /* the value of tile i and step t within a pair's reads */
   static OCH_SLAB_FN double value(const och_f64x2 (&f)[TILES], int i, int t) { return KC ? f[i][t] : f[t * (TILES / 2) + i / 2][i % 2]; }
   /* row (of the wave's rows) of tile i, row-in-tile rr */
   static OCH_SLAB_FN uint32_t row(int i, uint32_t rr) { return KC ? (uint32_t)i * 16 + rr : 32 * ((uint32_t)i / 2) + 2 * rr + (uint32_t)i % 2; }
};
} /* namespace och */
