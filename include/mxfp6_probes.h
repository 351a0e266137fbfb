/*
 * mxfp6_probes.h -- measurement entry points of the MI355X MXFP6 GEMM library, kept apart from the operator's ABI
 * (mxfp6_gemm.h).  They are exported by libmxfp6_probes.so only: a second build of the same sources with
 * -DMXFP6_PROBES, which adds the probe kernels, the ablation builds of the LDS-tiled kernel and the clock stamps in its
 * argument struct.  That library also exports everything mxfp6_gemm.h declares, so that a benchmark can time the same
 * calls with and without an override; the operator's own library carries none of this.  No counterpart in the reference.
 */
#ifndef MXFP6_PROBES_H
#define MXFP6_PROBES_H

#include <stddef.h>

#include "mxfp6_gemm.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * mxfp6_probe_mfma: a kernel that only issues v_mfma_scale_f32_32x32x64_f8f6f4 -- two waves per SIMD, each with two
 * fragments of A and two of B taken once from the given packed operands and scales (rows >= 32, K >= 64) and four
 * independent accumulators, `iters` rounds of four MFMAs.  Returns the number of waves launched (> 0; each issues
 * 4 * iters MFMAs of 131072 flop), or a negative MXFP6_E* code, or -(1000 + hipError_t).  stats[0..3] receive the shader
 * clock counter and the 100 MHz real-time counter of one workgroup at its start and end: clocks / time is the clock the
 * chip sustains under this load.  sink: one float of device memory (never written in practice).
 *
 * mxfp6_probe_stream: `workgroups` workgroups of `waves` (4 or 8) waves read `bytes` bytes (a multiple of
 * workgroups * waves * 8192) once, each wave a private contiguous range, through direct-to-LDS loads with 16 KB in flight
 * per wave, and do nothing else.  stats as above.
 *
 * mxfp6_probe_tiled_clock: per calling thread; while `stamps` is not NULL the LDS-tiled GEMM kernel's workgroup 0 writes
 * the same four counters (start, end) there on every launch.
 */
int mxfp6_probe_mfma(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale, int rows_a,
                     int rows_b, int K, int fmt_a, int fmt_b, int iters, float *sink, uint32_t *stats, void *hip_stream);
int mxfp6_probe_stream(const void *buf, size_t bytes, int workgroups, int waves, uint32_t *stats, void *hip_stream);
int mxfp6_probe_tiled_clock(uint32_t *stamps);

/*
 * The workgroup -> output tile map of the LDS-tiled kernel, evaluated on the host with the kernel's own function:
 * order[b] = pm | pn << 16 is the tile (row pm, column pn of a tiles_m x tiles_n grid) that logical workgroup b works on.
 * The kernel uses group_m = 4 and xcd_remap = 1; mxfp6_probe_raster (per calling thread, measurement only; group_m = 0
 * restores the default) makes later launches use other values, for sweeps of the raster like the reference's
 * (analysis/paper_experiments/grid_micro/data_to_log.json; remap include/common/util.cuh:78-101).  A host-side pointer:
 * `order` holds tiles_m * tiles_n ints.  Launches with a K split between workgroups order (tile, share) pairs share by
 * share and hand each XCD an eighth of that order, so that an XCD's workgroups work on one K range of A and B;
 * mxfp6_probe_raster(group_m, 2) keeps the tile remap but orders them tile by tile (measurement: the order before).
 */
int mxfp6_tile_order(int tiles_m, int tiles_n, int group_m, int xcd_remap, int *order);

/*
 * Ablations of the LDS-tiled kernel (per calling thread, measurement only, 0 = off): while mask != 0, e2m3 x e2m3 bf16
 * GEMMs on 256 x 256 tiles run a build of the kernel without its LDS reads of the operands (bit 0), without its
 * direct loads after the prologue (bit 1), without its MFMAs (bit 2); other calls fail with hipErrorInvalidValue.  The
 * output of such a launch is meaningless.  Timing the combinations 1 - 4 and 6 next to the full kernel (with
 * mxfp6_probe_tiled_clock for the shader clock) shows what each part costs and which ones the power management charges
 * (5 and 7, no LDS reads and no MFMAs at once, are not built and rejected: those builds spill registers).  mask = 8 is the
 * whole kernel with idle clocks added (every wave sleeps 128 clocks after every fourth MFMA; the output stays correct): if
 * the launch takes as long as without them while the shader clock rises, time is set by the power budget and not by the
 * schedule's clocks.
 */
int mxfp6_probe_tiled_ablation(int mask);
int mxfp6_probe_raster(int group_m, int xcd_remap);

/* The split the automatic path (shares = 0) or a forced setting would use for a shape on the current device: workgroups per
 * output tile (1 = none; negative = error code), and in *tile_rows (may be NULL) the rows of A per output tile (0 = none).
 * layouts: bit 0 set = A tile-major, bit 1 set = B tile-major (the e2m3 x e2m3 formats are assumed; the plan does not depend
 * on them). */
int mxfp6_probe_ksplit_plan(int M, int N, int K, int layouts, int shares, int *tile_rows);

/* Times a GEMM as the library would run it under this thread's mxfp6_set_kernel / mxfp6_set_k_split settings: `warmup`
 * untimed and `reps` timed back-to-back launches between two events on `hip_stream`, mean microseconds per launch in *us.
 * Launch i takes its B operand and B scales from B + (i % b_sets) * b_stride and Bs + (i % b_sets) * bs_stride (bytes), so that
 * a caller can rotate through more weights than the last-level cache holds, as a model's layers do.  Synchronises the
 * stream.  bf16 output unless out_f32.  The calibration sweep of the kernel choice and its checks time with this (no
 * interpreter between the launches: shapes of a few microseconds are timed on the GPU's side, as a replayed graph runs them). */
int mxfp6_probe_time_gemm(const void *A, const void *B, const void *A_scale, const void *B_scale, void *C, int M, int N, int K,
                          int fmt_a, int fmt_b, int layout_a, int layout_b, int out_f32, int b_sets, size_t b_stride,
                          size_t bs_stride, int warmup, int reps, double *us, void *hip_stream);

/* The kernel choice's view of one candidate on a shape (e2m3 x e2m3, bf16 output, 16-byte aligned tensors): *model_us is the
 * structural time model's figure in microseconds (negative: the candidate does not take the shape), *calibrated_us that figure
 * times the calibration factor of the nearest calibrated shape (what the choice compares), *shares the K split the candidate
 * would run with under the thread's mxfp6_set_k_split setting.  candidate: 0 - 2 the tiled kernel with tiles of 256 x 256 /
 * 128 x 256 / 128 x 128, 3 block, 4 block with tiles of 128 x 256, 5 skinny, 6 / 7 the tiled kernel's K split with tiles of
 * 256 / 128 rows, 8 the block kernel's K split, 9 ring.  cus: compute units to plan for (0 = the current device's).  Pure host code: the calibration tool
 * (python -m hipkittensp_amd.calibrate) calls it to turn a sweep's measured times into the table's factors. */
int mxfp6_probe_candidate(int M, int N, int K, int layouts, int candidate, int cus, double *model_us, double *calibrated_us,
                          int *shares);

/* Measurement switch, per calling thread: 0 keeps the block kernel (mxfp6_set_kernel 22 - 27) out of the automatic choice,
 * so that the same call can be timed with and without it; returns the previous setting.  Default 1. */
int mxfp6_probe_block(int enable);

#ifdef __cplusplus
}
#endif

#endif /* MXFP6_PROBES_H */
