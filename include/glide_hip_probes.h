/* Measurement yardsticks (libglide_probes.so).  NOT part of the drop-in boundary and without counterpart in the
 * reference: a maintainer binds nothing from this file.  bench.py's calibration flags use them to scale hardware
 * counters and to state the issue rates that counter readings of the product's kernels are held against. */
#ifndef GLIDE_HIP_PROBES_H
#define GLIDE_HIP_PROBES_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* A plain copy kernel (bytes % 16 == 0, 16-byte aligned): the transfer of known size against which hardware byte
 * counters (FETCH_SIZE / WRITE_SIZE) are calibrated.  Returns 0 or a negative glide_hip status / hipError. */
int glide_probe_copy_bytes(void *dst, const void *src, size_t bytes, void *stream);
/* A register-only kernel of 2048 x 256 threads, each running rounds x 16 independent steps: the yardstick for the
 * vector-ALU issue rate against which the instruction counters of the build and search kernels are read.
 * mode 0: fused multiply-add, 1: integer add, 2: compare + select (two instructions a step), 3: DPP cross-lane
 * move + add (two a step).  out: one float. */
int glide_probe_valu(int mode, uint32_t rounds, float *out, void *stream);
/* 2048 x 256 threads, each issuing `rounds` atomic operations on pseudo-random 8-byte slots of `table` (`slots` of
 * them, a power of two; the caller sets the table's contents): the yardstick for the rate of scattered atomics against
 * which the NN-descent kernels' offers and slot reservations are read.  mode 0: 64-bit minimum without a returned
 * value, 1: 32-bit add whose result is used, 2 / 3: as 0 with 2 / 16 adjacent lanes on slots of one 128-byte line.
 * out: one u32. */
int glide_probe_atomic(int mode, unsigned long long *table, uint32_t slots, uint32_t rounds, uint32_t *out,
                       void *stream);

/* `waves` wavefronts, each reading `rows_per_wave` pseudo-random rows of `row_bytes` (a multiple of 16) out of a table of
 * `row_count` rows that start `row_stride_bytes` apart, with 16-byte loads of adjacent lanes and nothing else to do: the rate at which scattered rows can be
 * fetched at all, the yardstick for the search kernels' row gathers.  rows_per_step 8 / 2 / 1: a row is read by 8 / 32 /
 * 64 lanes (the search kernels' shapes for 128-dim and 960-dim rows; one row per wavefront), with 16 / 8 / 8 rows requested
 * before the first is consumed.  out: one float. */
int glide_probe_gather(const void *table, uint32_t row_count, uint32_t row_bytes, uint32_t row_stride_bytes, uint32_t waves,
                       uint32_t rows_per_wave, int rows_per_step, float *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GLIDE_HIP_PROBES_H */
