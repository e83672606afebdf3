/*
 * oslo_hip_testing.h -- entry points of liboslo_hip.so that exist for the
 * test-suite, the benchmark and tuning sweeps only.  They have no counterpart
 * in the reference and are not part of the drop-in surface (oslo_hip.h):
 * production callers do not need them, and oslo_tune changes process-wide
 * state, which the production entry points never do.
 */
#ifndef OSLO_HIP_TESTING_H
#define OSLO_HIP_TESTING_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Raw Philox4x32-10 words: out[4*i .. 4*i+3] for counter
 * (offset_lo, offset_hi, group_lo, group_hi), group = first_group + i.     */
int oslo_philox_words(uint32_t *out, int64_t ngroups, int64_t first_group,
                      uint64_t seed, uint64_t offset, void *stream);

/* Plain device copy of `bytes` (multiple of 16) with the same 128-bit
 * load/store path the kernels use; calibrates bandwidth and HBM counters. */
int oslo_copy_probe(const void *src, void *dst, int64_t bytes, void *stream);

/* Measurement of a backward pass whose second launch runs beside other work:
 * with the knob "colsum_defer" set to 1 (oslo_tune) the backward entry points
 * that end in a column-sum launch (LayerNorm / RMSNorm, bias-GeLU,
 * bias-dropout-add and its fusion into the norm) stop after their main kernel
 * and leave the fp32 partial rows in the workspace: `parts` rows of `cols`
 * values per output; parts = workspace bytes / (outputs * cols * 4) for the
 * shapes the hook is meant for (long rows and at least as many rows as the
 * GPU has compute units; other shapes may fill fewer partial rows).  This
 * call then reduces them to out0 (and out1, out2) of `dtype`, on any stream. */
int oslo_colsum_finalize_probe(const void *partial_rows, int64_t parts, int64_t cols,
                               void *out0, void *out1, void *out2, int dtype,
                               void *stream);

/* Wavefront reduction self-test: out[0..3] = (sum, max, sum-of-pair a,
 * sum-of-pair b) of lane-dependent values; the expected values are
 * 2016, 63, 2016, 4032.                                                    */
int oslo_wave_reduce_selftest(float *out4, void *stream);

/* FOR TESTS AND TUNING SWEEPS ONLY, not for production callers: overrides a
 * launch heuristic; key is one of
 * "norm_fwd_vpl", "norm_bwd_vpl", "norm_bwd_blocks_per_cu", "norm_bwd_waves",
 * "norm_fwd_waves", "norm_bwd_prefetch", "norm_fwd_iters",
 * "norm_lanes_per_row", "softmax_lanes_per_row" (64 switches the
 * side-by-side short rows off, 1 the two-chunks-per-lane forward), "softmax_rows_per_wave", "softmax_rows_per_block" (rows, or sets of side-by-side rows, per workgroup: 1..16),
 * "softmax_fwd_elems", "eltwise_unroll", "eltwise_rowgroups",
 * "eltwise_fwd_steps", "eltwise_tile_max", "eltwise_tile_min" (lanes along
 * the columns of an element-wise tile; 64 as the minimum restores whole-wave
 * tiles), "adam_unroll", "softmax_bias_order" (order of the rows of a
 * softmax whose additive term is shared by the batch: 1 as stored, 2 the batch
 * entries of a run of rows of the term next to each other, the default, 3 that
 * and every eighth workgroup on consecutive rows), "softmax_bias_group" (rows
 * in such a run, a power of two up to 256, default 32; lowered to a divisor of
 * heads * queries), "softmax_causal_order" (order
 * of the queries of an attention matrix under the diagonal: 1 long rows first,
 * the default for rows of one wave, 2 as stored, the default for longer rows,
 * 3 long and short rows in turn), "colsum_defer" (1: see
 * oslo_colsum_finalize_probe), "colsum_slices" (slices of the partial rows
 * that a workgroup of the column-sum reduction adds side by side: 64 or 128,
 * the default, with eight lanes per slice and 32 columns per workgroup, or
 * 256 with four lanes per slice and 16 columns);
 * value 0 restores the default.  Other values must be ones the launch code
 * has a kernel build and a valid workgroup shape for, else
 * OSLO_ERR_INVALID_ARGUMENT: chunks per lane (*_vpl: 1, 2, 4, forward also 8,
 * and 3 for LayerNorm),
 * waves per workgroup 1..16, norm_bwd_prefetch 1 or 2, norm_fwd_iters 1..16,
 * norm_bwd_blocks_per_cu 1..8, lanes per row 8, 16, 32 or 64 (softmax also
 * 1), softmax_rows_per_wave and the unroll factors 1, 2 or 4 (eltwise_unroll
 * also 8, which only the bias-GeLU backward has a build for; the other
 * element-wise kernels then keep their default),
 * softmax_fwd_elems 16, 32 or 64, eltwise tile widths powers of two up to
 * 256, eltwise_rowgroups 1..4096, eltwise_fwd_steps 1..64.
 * The table is process-wide and written under a lock; every entry point
 * copies it once when it is called, so a launch never sees a half-changed
 * table, but calls that are already planned keep the old values.  No
 * accepted value changes a result beyond the order of summation.           */
int oslo_tune(const char *key, int value);

#ifdef __cplusplus
}
#endif
#endif /* OSLO_HIP_TESTING_H */
