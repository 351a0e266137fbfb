/*
 * mxfp6_gemm.h -- C ABI of the MI355X (gfx950) MXFP6 block-scaled GEMM.
 *
 *   C[M,N] = dq(A)[M,K] . dq(B)[N,K]^T        fp32 accumulation, bf16 (or fp32) output
 *
 * Operands are packed fp6 (e2m3 or e3m2, chosen per operand): row-major, K contiguous, value j of
 * a row at bits [6j, 6j+6) of the row's little-endian bitstream (4 values per 3 bytes, so a row is
 * 3K/4 bytes and a 32-element block is 24 contiguous bytes).  Each 32-element K-block of each row
 * carries one E8M0 scale byte (value 2^(b-127)); scale tensors are row-major [rows, K/32] uint8.
 *
 * This is the library a binding replaces the reference's per-kernel pybind module with.  The
 * reference convention it follows (benenzhu/HipKittensP):
 *   - entry point dispatch_micro(A, B, C): tensors in, C written in place, returns nothing,
 *     asynchronous launch, caller synchronises          analysis/bf16_gemm/mi325x/kernel_8192.cpp:227-237
 *   - C = A . B^T with both operands K-contiguous        kernels/gemm/bf16fp32/utils.py:28-37
 *   - tensor -> raw pointer conversion at the boundary   include/pyutils/pyutils.cuh:15-72
 * All pointers are DEVICE pointers.  All functions return 0 on success, a negative MXFP6_E* code
 * for rejected arguments (nothing launched), or a positive hipError_t value if the runtime failed.
 * Work is queued on `hip_stream` (a hipStream_t; NULL = the null stream); no function synchronises the
 * device or the stream.
 *
 * Device memory.  Four uses take a workspace from the stream-ordered allocator
 * (hipMallocAsync on `hip_stream`), at most once per (device, stream) and use (regrown when a later call
 * needs more), and keep it until mxfp6_release_workspaces():
 *   - the gemm entry points on large row-major problems (re-layout pre-pass, see mxfp6_set_relayout):
 *     up to 0.78 (M + N) K bytes;
 *   - mxfp6_gemm_fused_fp6 on shapes the LDS-tiled kernel does not run: 4 M N bytes;
 *   - the gemm entry points on decode shapes whose K range is split between workgroups (M <= 32, N <= 2048,
 *     K >= 24576): 2 MB;
 *   - the gemm entry points on problems of few output tiles and long K (up to a few hundred rows of A; see
 *     mxfp6_set_k_split), where the LDS-tiled kernel, the block kernel or the ring kernel splits K between workgroups:
 *     shares * 4 M N bytes of partial sums (tiles times shares never exceed the CUs: at most 64 MB, 256 tiles of
 *     256 x 256 fp32), one workspace for the three kernels, and for the ring kernel one counter per output tile.
 * While `hip_stream` is being captured nothing is allocated: the pre-pass and the K splits are left out
 * (same results up to the order of fp32 sums, other kernels) unless their workspace exists already, and mxfp6_gemm_fused_fp6 returns
 * hipErrorStreamCaptureUnsupported where it would need a new one.  A workspace that a capture did use is recorded in the
 * graph: the library never frees such a block again (when a later call needs a larger one, or at
 * mxfp6_release_workspaces(), it is kept allocated until the process ends), so the graph stays valid.  Replay it on the
 * stream it was captured on, or on another one only while no call of this library runs on the capture stream: the
 * replays and those calls share the workspace.  At most 128 workspaces exist at a time; beyond that the least recently
 * used one that no graph holds is returned to the allocator on its own stream, so call mxfp6_release_workspaces()
 * before destroying streams this library has seen.  mxfp6_gemm_noalloc never allocates.
 *
 * Alignment.  Pointers are accepted from 4-byte alignment on (C: its element size).  The fast kernels
 * fetch 16 bytes per lane: they run when A_packed, B_packed, both scale tensors and C are 16-byte aligned
 * (any tensor PyTorch allocates is); otherwise the call is served by the generic kernel, with the same
 * results and a fraction of the speed.
 *
 * Accuracy.  Products of dequantised values are exact in fp32; with an e2m3 operand on either side the
 * accumulators agree with an fp64 dequantise-and-matmul to fp32 rounding (relative error < 1e-6 of the
 * result's range).  e3m2 x e3m2 is weaker: the scaled MFMA's internal sum drops low-order bits of
 * wide-ranging products, giving an error of up to 1e-4 of sum_k |a_mk| |b_nk| per output, which is above
 * 2e-3 of the result only where the sum cancels to less than 5 % of its terms.  Because that can exceed the library's
 * stated bar without any sign, the gemm entry points return MXFP6_EACCURACY for that pair of formats until the calling
 * thread has accepted it with mxfp6_allow_e3m2_pair(1); every other pair meets the bar by construction.
 */
#ifndef MXFP6_GEMM_H
#define MXFP6_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* operand formats: the numbering of the scaled-MFMA format field */
#define MXFP6_FMT_E2M3 2
#define MXFP6_FMT_E3M2 3

#define MXFP6_OK 0
#define MXFP6_EINVAL_PTR (-1)   /* a required pointer is NULL                                  */
#define MXFP6_EINVAL_SHAPE (-2) /* M, N or K negative, K not a multiple of 32, or out of range */
#define MXFP6_EINVAL_FMT (-3)   /* format code is not 2 (e2m3) or 3 (e3m2)                     */
#define MXFP6_EINVAL_ALIGN (-4) /* a pointer violates the stated alignment                     */
#define MXFP6_ENODEVICE (-5)    /* current device is not gfx950                                */
#define MXFP6_EINVAL_LAYOUT (-6) /* layout code is not MXFP6_LAYOUT_ROW / MXFP6_LAYOUT_TILE    */
#define MXFP6_EINVAL_EPILOGUE (-7) /* activation code is not one of MXFP6_ACT_*                */
#define MXFP6_ESCRATCH (-8)     /* mxfp6_gemm_noalloc: the requested K split does not fit the static scratch memory */
#define MXFP6_EINVAL_KERNEL (-9) /* mxfp6_set_kernel: unknown kernel code                        */
#define MXFP6_EBLOB (-10)       /* not a tile-major operand blob of a version this library reads */
#define MXFP6_EACCURACY (-12)   /* e3m2 x e3m2 without mxfp6_allow_e3m2_pair(1): the pair can miss the 2e-3 accuracy bar */
#define MXFP6_EWORKSPACE (-11)  /* a call that cannot run without a workspace did not get one (allocator, or all slots held by graphs) */

/* Activations of mxfp6_gemm_fused. */
#define MXFP6_ACT_NONE 0
#define MXFP6_ACT_RELU 1
#define MXFP6_ACT_GELU 2 /* 0.5 y (1 + erf(y / sqrt 2)) */
#define MXFP6_ACT_SILU 3 /* y / (1 + exp(-y))           */

/*
 * The operator.  Replaces the reference's dispatch_micro(A, B, C) launcher
 * (analysis/bf16_gemm/mi325x/kernel_8192.cpp:227-231, distributed-kernels/bf16_gemm/kernel.cpp:247-265)
 * for packed-fp6 operands with E8M0 block scales.
 *   A_packed [M, 3K/4] u8, B_packed [N, 3K/4] u8, A_scale [M, K/32] u8, B_scale [N, K/32] u8,
 *   C [M, N] bf16 row-major.  K % 32 == 0.  A_packed/B_packed 4-byte aligned, C 2-byte aligned (16-byte
 *   alignment of all five tensors reaches the fast kernels, see "Alignment" above).
 *   M == 0 or N == 0 is a successful no-op; K == 0 writes zeros.
 */
int mxfp6_gemm(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale, void *C_bf16,
               int M, int N, int K, int fmt_a, int fmt_b, void *hip_stream);

/*
 * Same product with the fp32 accumulators stored unrounded (C is float [M, N]).  The accuracy
 * contract (max relative error vs the fp32 dequantise-and-matmul) is stated before the bf16
 * rounding, so this is the entry the parity tests measure; it shares every kernel with mxfp6_gemm.
 * Reference analogue: the float accumulator tile the reference converts at store time
 * (analysis/bf16_gemm/mi325x/kernel_8192.cpp:223-224).
 */
int mxfp6_gemm_f32out(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale,
                      float *C_f32, int M, int N, int K, int fmt_a, int fmt_b, void *hip_stream);

/*
 * Kernel selection override for measurement and tests, per calling thread (it affects the gemm calls this thread
 * makes afterwards, and nobody else's).  Returns the previous value, or MXFP6_EINVAL_KERNEL for an unknown code.
 * A forced kernel that cannot run the given shape makes the gemm calls return MXFP6_EINVAL_SHAPE.
 *    0  automatic (default)
 *    1  generic one-wave-per-tile kernel (any shape)
 *    2  LDS-tiled MFMA kernel (needs N % 8 == 0, K % 128 == 0), tile shape by how it fills the GPU;
 *       5 / 6 / 17: with output tiles of 128 x 256 / 256 x 256 / 128 x 128 (rows of A x rows of B)
 *    3  skinny-M streaming kernel (needs M <= 128, K % 512 == 0), workgroup geometry by N and K;
 *       7 / 8 / 9: 32 rows of B per workgroup / 16 rows / 32 rows and half the waves, none of them splitting K;
 *       10 / 11 / 12: 32 rows of B, the K range split between 2 / 4 / 8 workgroups; 13 / 14 / 15: the same with 16 rows
 *       (the split takes a workspace of 2 MB per stream at first use; without one, e.g. first use under stream capture,
 *       the launch runs unsplit); 16: 32 rows of B and two waves per workgroup;
 *       19 / 20 / 21: 64 rows of B per workgroup (two tiles of B against every fragment of A: half the bytes of A come
 *       from L2 per byte of B), the K range unsplit / split between 2 / 4 workgroups (the same workspace; a split whose partial
 *       tiles do not fit it runs unsplit)
 *    4  mid-M kernel (needs 32 < M <= 512, K % 1024 == 0, row-major A)
 *   18  the 4-wave interleaved schedule of the LDS-tiled kernel (one wave per SIMD with a 128 x 128 wave tile; shapes
 *       of kernel 2, no fused epilogue); never chosen automatically, kept to compare the two schedules
 *   28  ring kernel for batched decode (needs K % 512 == 0, N % 4 == 0): every wave streams its own 32 rows of B through
 *       private LDS slots, A comes through a ring that a loader wave fills and flags guard, no barrier per K-tile;
 *       splits K between workgroups by the thread's mxfp6_set_k_split setting
 *   22  block kernel: output tiles of 128 x 128, four waves in step with the operand fragments double-buffered in
 *       registers, one barrier per K-tile (needs N % 8 == 0, K % 128 == 0); typically chosen for a few hundred to a few
 *       thousand rows of A;
 *       23 / 24: with an operand ring of three slots (two workgroups per CU) / six slots (one); 26: with tiles of
 *       128 x 256 and eight waves.  22 - 24 split K between workgroups by the thread's mxfp6_set_k_split setting
 *       (0: where the library's time model prefers the split; the same per-stream workspace as the tiled kernel's split)
 * No counterpart in the reference, whose shapes are compile-time constants per binary
 * (analysis/bf16_gemm/mi350x/mi355x_benchmark.sh).
 */
int mxfp6_set_kernel(int which);

/*
 * Re-layout pre-pass of the automatic path (on by default; per calling thread; returns the previous setting).
 * For large row-major problems the gemm calls first copy one operand or both (with their scales) into
 * tile-major order in this stream's workspace (hipMallocAsync on the caller's stream the first time, kept
 * until mxfp6_release_workspaces()), because the tiled kernel is bound by L2 requests on row-major operands;
 * results are bit-identical.  On a stream that is being captured it runs only if the workspace exists already.
 * Switch it off to measure the row-major kernel itself.  No counterpart in the reference.
 */
int mxfp6_set_relayout(int on);

/*
 * Quantise + pack on the GPU: X [rows, K] fp32 row-major -> packed [rows, 3K/4] u8 + scales
 * [rows, K/32] u8, scale = 2^(floor(log2(blockmax)) - emax(fmt)) (emax 2 for e2m3, 4 for e3m2),
 * round-to-nearest-even, saturating; an all-zero block gets scale byte 0.  K % 32 == 0.
 * The producer of this path's inputs; the reference's harness creates its operands on the device
 * the same way (kernels/gemm/bf16fp32/utils.py:28-34).
 */
int mxfp6_quantize(const float *X, void *packed, void *scales, int rows, int K, int fmt, void *hip_stream);

/*
 * Tile-major operand layout ("pre-shuffled" operands; rows % 32 == 0, K % 128 == 0).  The packed bytes
 * of an operand are regrouped into tiles of 32 rows x 128 elements (3072 bytes), tile (rt, kt) at byte
 * ((rt * (K/128)) + kt) * 3072; inside a tile, the 16-byte piece c (0..5) of row r (0..31) sits at
 * (r*6 + (c ^ ((r >> 3) & 1))) * 16.  This is exactly the image the kernels keep in LDS, so their
 * direct-to-LDS loads become fully contiguous (one 1 KiB run per load instead of ~11 row pieces).
 * The scales of a tile-major operand are tile-major too: the 16 scale bytes one row has for four K-tiles
 * (512 elements) stay together and the 32 rows of a row-tile are adjacent, i.e. 512-byte chunk (rt, g) at
 * ((rt * nk4) + g) * 512 with nk4 = ceil(K / 512), the byte of K-block kb of row r at (r % 32) * 16 + kb % 16
 * inside chunk (r / 32, kb / 16).  The scale tensor then holds rows * nk4 * 16 bytes (= rows * K/32 when
 * K % 512 == 0; the bytes of K-blocks past K are padding).  A kernel's scale load of 32 rows is 4 cache
 * lines instead of 32.  The reference applies its LDS swizzle to the global address of every
 * load (include/ops/warp/memory/tile/global_to_shared.cuh:46-59); this applies it to the data once,
 * which suits weights (converted offline) and activations (the quantiser can emit it directly).
 */
#define MXFP6_LAYOUT_ROW 0  /* [rows, 3K/4], K contiguous: the layout of mxfp6_gemm                */
#define MXFP6_LAYOUT_TILE 1 /* tile-major, see above                                                */

/* Row-major packed operand -> tile-major (tile != 0) or back (tile == 0); src and dst must not overlap. */
int mxfp6_tile_operand(const void *src, void *dst, int rows, int K, int tile, void *hip_stream);

/*
 * Scales [rows, K/32] row-major -> tile-major (tile != 0; rows * ceil(K/512) * 16 bytes, padding written as 0)
 * or back (tile == 0); rows % 32 == 0, K % 128 == 0; src and dst must not overlap.  No counterpart in the
 * reference (its operands carry no scales); part of the tile-major operand format above.
 */
int mxfp6_tile_scales(const void *src, void *dst, int rows, int K, int tile, void *hip_stream);

/*
 * Serialised tile-major operand (a weight converted once, stored or shipped, and used without conversion): a blob of
 *   bytes  0 ..  3  magic "MX6T"
 *   byte   4        format version (1)
 *   byte   5        operand format (MXFP6_FMT_E2M3 / MXFP6_FMT_E3M2)
 *   byte   6        layout (MXFP6_LAYOUT_TILE)
 *   byte   7        reserved, 0
 *   bytes  8 .. 11  rows, bytes 12 .. 15  K   (little endian)
 *   then the tile-major packed bytes (rows * 3K/4) and the tile-major scales (rows * ceil(K/512) * 16), as defined above.
 * rows % 32 == 0, K % 128 == 0.  Both parts start 16-byte aligned inside a 16-byte aligned blob, so a blob in device
 * memory is used in place: blob + 16 and blob + 16 + rows * 3K/4 are the operand and scale pointers of mxfp6_gemm_ex with
 * MXFP6_LAYOUT_TILE.  mxfp6_blob_bytes: size of the blob (0 for a shape it cannot hold).  mxfp6_blob_header_write /
 * _read work on 16 bytes of HOST memory; _read returns MXFP6_EBLOB for a wrong magic, an unknown version, format or
 * layout, a non-zero reserved byte or an impossible shape.  mxfp6_blob_pack writes the whole blob, header included, in
 * DEVICE memory from a row-major operand and its row-major scales; mxfp6_blob_unpack converts a device blob's body back
 * (the caller has read rows and K from a host copy of the header).  No counterpart in the reference, which has no
 * stored operand format; the layout itself is the swizzle of include/ops/warp/memory/tile/global_to_shared.cuh:46-59
 * applied to the data.
 */
size_t mxfp6_blob_bytes(int rows, int K);
int mxfp6_blob_header_write(void *header16_host, int rows, int K, int fmt);
int mxfp6_blob_header_read(const void *header16_host, int *rows, int *K, int *fmt);
int mxfp6_blob_pack(const void *packed_row_major, const void *scales_row_major, void *blob, int rows, int K, int fmt,
                    void *hip_stream);
int mxfp6_blob_unpack(const void *blob, void *packed_row_major, void *scales_row_major, int rows, int K,
                      void *hip_stream);

/*
 * mxfp6_gemm / mxfp6_gemm_f32out with a layout per operand (MXFP6_LAYOUT_*) and out_f32 != 0 for
 * the fp32 output.  With both layouts MXFP6_LAYOUT_ROW it is exactly those two entry points.
 * A tile-major operand comes with tile-major scales and needs rows % 32 == 0 and K % 128 == 0
 * (MXFP6_EINVAL_SHAPE otherwise).
 */
int mxfp6_gemm_ex(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale, void *C,
                  int M, int N, int K, int fmt_a, int fmt_b, int layout_a, int layout_b, int out_f32,
                  void *hip_stream);

/* mxfp6_quantize writing the packed operand and its scales in the given layout (tile-major scales: rows *
 * ceil(K/512) * 16 bytes, of which the padding bytes are not written). */
int mxfp6_quantize_ex(const float *X, void *packed, void *scales, int rows, int K, int fmt, int layout,
                      void *hip_stream);

/* mxfp6_quantize_ex for bf16 input (X: rows x K bf16, 16-byte aligned): the values a float copy of X would give,
 * without the copy.  Activations of bf16 models are the usual input; no counterpart in the reference, whose
 * harness converts on the host side (kernels/gemm/bf16fp32/utils.py:28-34). */
int mxfp6_quantize_bf16(const void *X_bf16, void *packed, void *scales, int rows, int K, int fmt, int layout,
                        void *hip_stream);

/*
 * mxfp6_gemm_ex with work fused into the epilogue, in fp32 on the accumulators before the output rounding:
 *   C[m][n] = act(acc[m][n] * row_scale[m] * col_scale[n] + bias[n])
 * Every vector is optional (NULL = leave out): bias [N] float (bias_bf16 == 0) or bf16 (!= 0), row_scale [M]
 * float (e.g. a per-token activation scale), col_scale [N] float (e.g. a per-channel weight scale); activation
 * is one of MXFP6_ACT_*.  With everything left out it is mxfp6_gemm_ex.  Alignment: bias and col_scale 16
 * bytes (bf16 bias 8), row_scale 4.  gelu and silu are computed with the hardware exp2 / reciprocal and a
 * five-term erf (absolute error <= 1.5e-7): results agree with a double-precision evaluation to about 1e-6 of
 * the output range, not bit for bit.
 * No counterpart in the reference, whose GEMMs store the accumulator tile as it is
 * (analysis/bf16_gemm/mi325x/kernel_8192.cpp:223-224); it removes a pass over C for the usual linear-layer tail.
 */
int mxfp6_gemm_fused(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale, void *C,
                     int M, int N, int K, int fmt_a, int fmt_b, int layout_a, int layout_b, int out_f32,
                     const void *bias, int bias_bf16, const float *row_scale, const float *col_scale, int activation,
                     void *hip_stream);

/*
 * mxfp6_gemm_fused whose result is re-quantised to MXFP6 along N, i.e. written as the packed operand
 * C_packed [M, 3N/4] and its E8M0 scales C_scale [M, N/32] (row-major) that the next layer's GEMM takes as A:
 * exactly mxfp6_quantize(fmt_c) applied to the fp32 result of mxfp6_gemm_fused(out_f32 = 1), without that result
 * ever reaching memory (0.78 instead of 2 or 4 bytes per output element).  N % 32 == 0; C_packed 8-byte aligned.
 * The LDS-tiled kernel quantises its accumulators in its epilogue; shapes that run on another kernel (few rows of A,
 * where C is small) go through an fp32 workspace taken from and returned to the stream-ordered allocator on
 * hip_stream, and are refused under stream capture (hipErrorStreamCaptureUnsupported).
 * No counterpart in the reference.
 */
int mxfp6_gemm_fused_fp6(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale,
                         void *C_packed, void *C_scale, int M, int N, int K, int fmt_a, int fmt_b, int layout_a,
                         int layout_b, int fmt_c, const void *bias, int bias_bf16, const float *row_scale,
                         const float *col_scale, int activation, void *hip_stream);

/*
 * Returns every workspace this library holds (see "Device memory" above) to the stream-ordered allocator, each in
 * the order of the stream it was taken on; later calls allocate again on demand.  No counterpart in the reference,
 * which allocates nothing behind its launcher.
 */
int mxfp6_release_workspaces(void);

/*
 * mxfp6_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): same operands, same bf16 result, and no allocation of any kind.  It has no
 * counterpart in the reference.  The re-layout pre-pass is left out, and the K split of decode shapes keeps its partial
 * tiles (4 KB per tile of C and split) and arrival counters in a static array of the library's device code: 1 MB + 1 KB
 * per GPU, held until the process ends, holding 256 partial tiles and 256 counters.
 *   nsplit = 0: the kernel mxfp6_gemm would choose among those that need no workspace (the skinny, mid-M, tiled and
 *               generic kernels; the skinny kernel's K split as mxfp6_gemm chooses it, never more than 256 partial
 *               tiles).  Where that is mxfp6_gemm's own choice -- the decode shapes it gives to the skinny kernel --
 *               the result is bit-identical to mxfp6_gemm's, and so it is where mxfp6_gemm takes the pre-pass or
 *               the block kernel unsplit (the sum along K runs in the same order); where mxfp6_gemm takes a K split
 *               of the tiled or block kernel, or a kernel of another family for the shape, the same products are
 *               added in another order: equal within the rounding of fp32 partial sums, and bit-identical whenever
 *               those sums are exact;
 *   nsplit = 1: as nsplit = 0, but K is never split between workgroups (nothing touches the static array);
 *   nsplit = 2, 4, 8: the skinny kernel with K split between that many workgroups per tile of C (needs M <= 32,
 *               K % 512 == 0; MXFP6_EINVAL_SHAPE otherwise).  A tile of C is 16 columns for N <= 4096 and 32 beyond:
 *               ceil(N / 16 or 32) * nsplit must not exceed 256, else MXFP6_ESCRATCH and nothing is launched.
 * Every call on a GPU shares that GPU's array: the counters are cleared by a small kernel in front of each split launch,
 * and calls that overlap in time on one GPU (two streams, two threads) race on it -- serialise them, or give the
 * concurrent ones nsplit = 1.
 */
int mxfp6_gemm_noalloc(const void *A_packed, const void *B_packed, const void *A_scale, const void *B_scale,
                       void *C_bf16, int M, int N, int K, int fmt_a, int fmt_b, int nsplit, void *hip_stream);

/* e3m2 x e3m2 (see "Accuracy" above): 1 lets this thread's later gemm calls run that pair of formats, 0 (the default) makes
 * them return MXFP6_EACCURACY.  Returns the previous setting.  No counterpart in the reference. */
int mxfp6_allow_e3m2_pair(int allow);

/*
 * K split between workgroups (per calling thread; returns the previous setting).  Problems of few output tiles and long K
 * (up to a few hundred rows of A against a wide weight matrix) run with several workgroups per output tile, each over a
 * part of K.  The LDS-tiled and the block kernel's shares leave fp32 partial matrices in this stream's workspace and a
 * second small kernel adds them in share order and applies the epilogue; the ring kernel's shares leave partial tiles
 * there and the workgroup that arrives last at a tile adds them in share order.  Either way the result does not depend
 * on timing.  0 = where it pays (default), 1 = never, -1 = wherever the shape allows it, n > 1 = n workgroups per output
 * tile where the shape allows it, else unsplit.  No counterpart in the reference (its GEMMs are one workgroup per
 * 256 x 256 tile, analysis/bf16_gemm/mi325x/kernel_8192.cpp:45-61).
 */
int mxfp6_set_k_split(int shares);

/* The kernel the automatic path takes for a problem of this shape on the current device (e2m3 x e2m3, bf16 output, no fused
 * epilogue, 16-byte aligned tensors): a code of mxfp6_set_kernel, or 25 / 27 for the tiled / the block kernel with its
 * K split between workgroups; negative = error code.  layouts: bit 0 set = A tile-major, bit 1 set = B tile-major.
 * Reads the thread's mxfp6_set_k_split setting; launches nothing. */
int mxfp6_kernel_choice(int M, int N, int K, int layouts);

/* Human-readable text for a return code of this library (never NULL). */
const char *mxfp6_strerror(int code);

/* ABI version of this header, major * 100 + minor, and what the loaded library reports: a caller built against this
 * header checks that the majors agree (entry points are only ever added within a major). */
#define MXFP6_ABI_VERSION 200
int mxfp6_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MXFP6_GEMM_H */
