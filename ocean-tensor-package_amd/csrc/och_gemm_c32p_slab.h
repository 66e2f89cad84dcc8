/* Where the slabs of the pipelined complex-float GEMM (och_gemm_c32p.hip) lie in LDS; index arithmetic only, so that a host
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

#define OCH_CP_OPERAND 34816                 /* LDS bytes of one operand's slab, either layout */

namespace och {

typedef float och_f32x4 __attribute__((ext_vector_type(4)));

/* one operand's slab of 128 rows: where its loads come from and go to, where the fragments are read, which row a
   fragment value belongs to */
template <bool KC>
struct CFloatSlab
{
   static constexpr int PLANE = 128 * 16 + 128;      /* KC: bytes per chunk plane (16 chunks of 2 k) */
   static constexpr int ROWP = 128 * 8 + 64;         /* !KC: bytes per k */
   static_assert(16 * PLANE <= OCH_CP_OPERAND && 32 * ROWP <= OCH_CP_OPERAND, "slab does not fit");
   /* load j (0 .. 7) of wave w: byte offset in memory relative to the slab's first element, per lane. KC: chunk
      (w / 2) * 8 + j of the 64 rows of group w % 2; !KC: k = 8 w + j */
   /* `rows`: how many of the tile's rows exist (a multiple of 2; fewer than 128 in the last tile of a matrix whose size is
      not a multiple of the tile). Lanes whose rows do not exist fetch the last rows that do: loads stay inside the matrix,
      and what they bring is multiplied into rows of the tile that are never written. */
   static OCH_SLAB_FN uint32_t load_offset(int j, uint32_t wave, uint32_t lane, int64_t ld, uint32_t rows)
   {  if (KC)
      {  uint32_t row = (wave % 2) * 64 + lane;
         row = row < rows ? row : rows - 1;
         return (uint32_t)((int64_t)row * ld * 8 + ((wave / 2) * 8 + j) * 16);
      }
      uint32_t row = lane * 2;
      row = row < rows ? row : rows - 2;
      return (uint32_t)((int64_t)(wave * 8 + j) * ld * 8 + row * 8);
   }
   /* ... and its first byte in the operand's LDS area (lane l writes 16 bytes at + 16 l) */
   static OCH_SLAB_FN uint32_t load_target(int j, uint32_t wave)
   {  return KC ? ((wave / 2) * 8 + j) * PLANE + (wave % 2) * 1024 : (wave * 8 + j) * ROWP; }
   static OCH_SLAB_FN const char *slab_base(const char *mat, int64_t ld, uint32_t mn0, uint32_t k0)
   {  return mat + (KC ? ((int64_t)k0 + (int64_t)mn0 * ld) : ((int64_t)mn0 + (int64_t)k0 * ld)) * 8; }
   /* fragment read x (0 .. 3) of quad q -- read x % 2 of its pair x / 2: the lane's part of the address, and the immediate part */
   static OCH_SLAB_FN uint32_t read_lane(uint32_t wbase, uint32_t lane)
   {  const uint32_t r = lane % 32, kg = lane / 32;
      return KC ? kg * PLANE + (wbase + r) * 16 : 2 * kg * ROWP + (wbase + 2 * r) * 8;
   }
   static constexpr uint32_t read_offset(int x, int q)
   {  return KC ? (uint32_t)(2 * (2 * q + x / 2) * PLANE + (x % 2) * 32 * 16) : (uint32_t)((4 * (2 * q + x / 2) + x % 2) * ROWP); }
   /* part c (0: real, 1: imaginary) of the value of tile i in step t (0 .. 3) within a quad's four reads */
   static OCH_SLAB_FN float value(const och_f32x4 (&f)[4], int i, int t, int c)
   {  return KC ? f[2 * (t / 2) + i][2 * (t % 2) + c] : f[2 * (t / 2) + t % 2][2 * i + c]; }
   /* row (of the wave's 64) of tile i, row-in-tile rr */
   static OCH_SLAB_FN uint32_t row(int i, uint32_t rr) { return KC ? (uint32_t)i * 32 + rr : 2 * rr + (uint32_t)i; }
};

} /* namespace och */
