/* Where the slabs of the pipelined complex-double GEMM (och_gemm_c64p.hip) lie in LDS; index arithmetic only, so that a host
   program can walk through it (tests/gemm_slab_host.cpp). */
#pragma once
#include <stdint.h>

#ifndef OCH_SLAB_FN
#  if defined(__HIPCC__)
#     define OCH_SLAB_FN __host__ __device__ __forceinline__
#  else
#     define OCH_SLAB_FN inline
#  endif
#endif

#define OCH_ZP_KT 16

namespace och {

typedef double och_f64x2 __attribute__((ext_vector_type(2)));

/* one operand's slab of ROWS = 128 or 64 rows and 16 k, [k][row][re, im] in LDS: where its loads come from and go to,
   where the fragments are read */
template <bool KC, int ROWS>
struct CDoubleSlab
{
   static constexpr int PLANE = ROWS * 16 + 64;      /* bytes per k */
   static constexpr int LOADS = ROWS * OCH_ZP_KT * 16 / 1024 / 4;     /* loads per wave and slab: 8 or 4 */
   static constexpr int TILES = ROWS / 2 / 16;       /* tiles per wave: 4 or 2 */
   static constexpr int READS = 2 * TILES;           /* fragment reads per pair of steps */
   static constexpr int PARTS = ROWS / 64;           /* groups of 64 rows: one load instruction each per k */
   /* load j of wave w: unit u = w * LOADS + j is the rows 64 (u % PARTS) ... of k = u / PARTS; lane l fetches row l of them.
      `rows`: how many of the tile's rows exist; lanes whose row does not exist fetch the last one that does */
   static OCH_SLAB_FN uint32_t load_offset(int j, uint32_t wave, uint32_t lane, int64_t ld, uint32_t rows)
   {  const uint32_t u = wave * LOADS + j, k = u / PARTS;
      uint32_t row = (u % PARTS) * 64 + lane;
      row = row < rows ? row : rows - 1;
      return (uint32_t)((KC ? (int64_t)row * ld + k : (int64_t)k * ld + row) * 16);
   }
   static OCH_SLAB_FN uint32_t load_target(int j, uint32_t wave)
   {  const uint32_t u = wave * LOADS + j;
      return (u / PARTS) * PLANE + (u % PARTS) * 1024;
   }
   static OCH_SLAB_FN const char *slab_base(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0)
   {  return mat + (KC ? ((int64_t)k0 + (int64_t)mn0 * ld) : ((int64_t)mn0 + (int64_t)k0 * ld)) * 16; }
   /* fragment read x (0 .. READS - 1) of pair P -- tile x % TILES in step x / TILES: the lane's part of the address, and the immediate part */
   static OCH_SLAB_FN uint32_t read_lane(uint32_t wbase, uint32_t lane)
   {  const uint32_t r = lane % 16, kg = lane / 16;
      return kg * PLANE + (wbase + r) * 16;
   }
   static constexpr uint32_t read_offset(int x, int P) { return (uint32_t)(4 * (2 * P + x / TILES) * PLANE + (x % TILES) * 256); }
   /* part c (0: real, 1: imaginary) of the value of tile i in step t within a pair's reads */
   static OCH_SLAB_FN double value(const och_f64x2 (&f)[READS], int i, int t, int c) { return f[t * TILES + i][c]; }
   /* row (of the wave's rows) of tile i, row-in-tile rr */
   static OCH_SLAB_FN uint32_t row(int i, uint32_t rr) { return (uint32_t)i * 16 + rr; }
};
} /* namespace och */
