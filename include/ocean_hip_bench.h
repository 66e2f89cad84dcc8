/* ------------------------------------------------------------------------ */
/* ocean_hip_bench.h -- the two micro-benchmarks that the library's own     */
/* measurements are set against (bench.py): what the device sustains from   */
/* memory for the traffic mixes of the streaming kernels, and what its       */
/* matrix cores sustain in a loop of nothing but MFMAs. They are measurement */
/* tools, built into a library of their own (csrc/libocean_hip_bench.so,     */
/* which uses libocean_hip.so for its error reporting); the product ABI is   */
/* include/ocean_hip.h alone. Neither has a counterpart in the reference.    */
/* ------------------------------------------------------------------------ */
#ifndef OCEAN_HIP_BENCH_H
#define OCEAN_HIP_BENCH_H
#include "ocean_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Streaming micro-benchmark (no counterpart in the reference): what the device sustains for the traffic mixes of   */
/* the elementwise / copy / cast kernels, measured with plain kernels that do nothing else. kind: 0 read, 1 write,  */
/* 2 copy, 3 add of doubles (2 reads : 1 write), 4 float -> double (4 B read : 8 B written), 5 every second int16   */
/* -> float, 6 / 7 other forms of 4 / 5. nbytes = bytes of the narrowest operand per launch. unr (1, 2, 4) = groups */
/* in flight per thread; nt = nontemporal hint;                     map 0 = one trip per thread, 1 = persistent    */
/* grid of `blocks` blocks walking contiguous ranges; block = threads per workgroup. The call allocates `nsets`     */
/* operand sets (rotated between launches so that nothing is served from the last-level cache), fills them with     */
/* pseudo-random bits, times `reps` samples of ten back-to-back launches with events on `stream`, frees everything, */
/* and returns the median and best time of one launch and the bytes one launch moves. Synchronous.                  */
int och_membench(int kind, int unr, int nt, int map, int block, int blocks, size_t nbytes, int nsets, int reps,
                 float *median_ms, float *best_ms, size_t *bytes_moved, och_stream stream);

/* Matrix-core micro-benchmark (no counterpart in the reference): the rate of a loop of nothing but MFMAs, and what     */
/* other instructions of the same wave cost between them. type: 0 float 32x32x2, 1 double 16x16x4, 2 half 32x32x16,    */
/* 3 int8 32x32x32. kind: 0 MFMAs alone on 16 pseudo-random operand pairs in turn, 7 MFMAs alone on one operand pair   */
/* (the power drawn, and with it the clock, depends on it), 1 v_mov_b32, 2 v_add_f32, 3 s_nop, 4 s_add_u32, 5 s_waitcnt, 6 ds_read_b128, */
/* `per_mfma` (1, 2 or 4) of them after every MFMA. waves: 4 or 8 per block, one block per compute unit. Times `reps`  */
/* launches of `iters` iterations of 16 MFMAs per wave with events on `stream`; returns the median time of a launch    */
/* and the flop (or integer operations) it performs. Allocates and frees its own small buffers. Synchronous.           */
int och_mfmabench(int type, int kind, int per_mfma, int waves, int iters, int reps, float *median_ms, double *flop, och_stream stream);

#ifdef __cplusplus
}
#endif
#endif
