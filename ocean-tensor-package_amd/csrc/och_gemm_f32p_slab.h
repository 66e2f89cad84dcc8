/* Where the slabs of the pipelined float GEMM (och_gemm_f32p.hip) lie in LDS: which bytes a load instruction of a wave
   fetches and where it puts them, where a lane reads its fragments, and which row and k of the operand a fragment value
   is. Index arithmetic only, so that a host program can walk through it (tests/gemm_slab_host.cpp builds a slab in
   ordinary memory with these functions and checks that every MFMA operand is the matrix element it has to be). */
#pragma once
#include <stdint.h>

#ifndef OCH_SLAB_FN
#  if defined(__HIPCC__)
#     define OCH_SLAB_FN __host__ __device__ __forceinline__
#  else
#     define OCH_SLAB_FN inline
#  endif
#endif

namespace och {

typedef float och_f32x4 __attribute__((ext_vector_type(4)));
typedef float och_f32x2 __attribute__((ext_vector_type(2)));

/* one operand's slab of ROWS = 256, 128 or 64 rows: where its loads come from and go to, where the fragments are read, which
   row a fragment value belongs to. TS = ROWS / 64 tiles of 32 rows per wave. */
template <bool KC, int ROWS>
struct FloatSlab
{
   static constexpr int TS = ROWS / 64;
   static constexpr int PLANE = ROWS * 16 + 128;     /* KC: bytes per chunk plane; the odd 32 banks keep the two lane halves apart */
   static constexpr int KPI = 256 / ROWS;            /* !KC: k per load instruction (1 KB of rows) and ... */
   static constexpr int UNIT = 1024 + 32 * KPI;      /* ... bytes from one instruction's rows to the next one's */
   static constexpr int OPERAND = 8 * PLANE;         /* LDS bytes of the slab, either layout */
   static_assert((32 / KPI) * UNIT <= OPERAND, "slab does not fit");
   static constexpr int LOADS = ROWS / 32;           /* loads per wave and slab */
   static constexpr int GROUPS = ROWS / 64;          /* KC: groups of 64 rows, one row per lane */
   static constexpr int READS = KC ? TS : 4;         /* fragment reads per quad */
   static constexpr uint32_t k_offset(int k) { return (uint32_t)((k / KPI) * UNIT + (k % KPI) * ROWS * 4); }      /* !KC: where k starts */
   /* load j of wave w: byte offset in memory relative to the slab's first element, per lane. KC: chunk (w / GROUPS) * LOADS + j
      of the rows of group w % GROUPS; !KC: k = (w * LOADS + j) * KPI + lane / (64 / KPI), 16 bytes of rows per lane */
   /* `rows`: how many of the tile's rows exist (a multiple of 4; fewer than ROWS in the last tile of a matrix whose size is
      not a multiple of the tile). Lanes whose rows do not exist fetch the last rows that do: loads stay inside the matrix,
      and what they bring is multiplied into rows of the tile that are never written. */
   static OCH_SLAB_FN uint32_t load_offset(int j, uint32_t wave, uint32_t lane, int64_t ld, uint32_t rows)
   {  if (KC)
      {  uint32_t row = (wave % GROUPS) * 64 + lane;
         row = row < rows ? row : rows - 1;
         return (uint32_t)((int64_t)row * ld * 4 + ((wave / GROUPS) * LOADS + j) * 16);
      }
      constexpr uint32_t LPK = 64 / KPI;
      uint32_t row = (lane % LPK) * 4;
      row = row < rows ? row : rows - 4;
      return (uint32_t)((int64_t)((wave * LOADS + j) * KPI + lane / LPK) * ld * 4 + row * 4);
   }
   /* ... and its first byte in the operand's LDS area (lane l writes 16 bytes at + 16 l) */
   static OCH_SLAB_FN uint32_t load_target(int j, uint32_t wave)
   {  return KC ? ((wave / GROUPS) * LOADS + j) * PLANE + (wave % GROUPS) * 1024 : (wave * LOADS + j) * UNIT; }
   static OCH_SLAB_FN const char *slab_base(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0)
   {  return mat + (KC ? ((int64_t)k0 + (int64_t)mn0 * ld) : ((int64_t)mn0 + (int64_t)k0 * ld)) * 4; }
   /* fragment read x (0 .. READS - 1) of quad q: the lane's part of the address, and the immediate part */
   static OCH_SLAB_FN uint32_t read_lane(uint32_t wbase, uint32_t lane)
   {  const uint32_t r = lane % 32, kg = lane / 32;
      return KC ? kg * PLANE + (wbase + r) * 16 : kg * k_offset(4) + (wbase + TS * r) * 4;
   }
   static constexpr uint32_t read_offset(int x, int q) { return KC ? (uint32_t)(2 * q * PLANE + x * 32 * 16) : k_offset(8 * q + x); }
   /* KC: the four steps of one tile, 16 bytes; !KC: the TS tiles of one step, 4 TS bytes */
   static OCH_SLAB_FN och_f32x4 read(const char *at)
   {  if (KC || TS == 4) return *reinterpret_cast<const och_f32x4 *>(at);
      if (TS == 1) return och_f32x4{*reinterpret_cast<const float *>(at), 0.0f, 0.0f, 0.0f};
      const och_f32x2 v = *reinterpret_cast<const och_f32x2 *>(at);
      return och_f32x4{v.x, v.y, 0.0f, 0.0f};
   }
   /* the value of tile i and step t within a quad's reads */
   static OCH_SLAB_FN float value(const och_f32x4 (&f)[4], int i, int t) { return KC ? f[i][t] : f[t][i]; }
   /* row (of the wave's 32 TS) of tile i, row-in-tile rr */
   static OCH_SLAB_FN uint32_t row(int i, uint32_t rr) { return KC ? (uint32_t)i * 32 + rr : TS * rr + (uint32_t)i; }
};

} /* namespace och */
