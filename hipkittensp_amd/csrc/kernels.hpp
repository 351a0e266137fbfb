// Internal launcher interface between the C ABI (api.hip) and the kernel translation units.
#pragma once
#include "common.hpp"
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mxfp6 {

struct GemmArgs {
  const uint8_t *A, *B, *As, *Bs;  // packed operands and E8M0 scales (device)
  void* C;                         // bf16 or float [M, N]
  int M, N, K;
  int fmt_a, fmt_b;  // 2 = e2m3, 3 = e3m2
  bool f32out;
  int layout_a = 0, layout_b = 0;  // 0 = row-major, 1 = tile-major (operand: 32 rows x 128 elements in LDS image order; scales: 32 rows x 16 bytes)
  int tile_rows = 0;               // tiled kernel: rows of A per output tile, 128 or 256; 0 = chosen per shape
  int tile_cols = 0;               // ... and rows of B: 128 (with 128 rows of A only) or 256; 0 with tile_rows set = 256
  int skinny_geometry = 0;         // skinny kernel: 1 = 32 rows of B and all waves, 2 = 16 rows of B, 3 = half the waves, 4 - 9 = 1 or 2 with the K range split between 2 / 4 / 8 workgroups, 10 = two waves; 0 = by shape
  Epilogue ep;                     // fused bias / scales / activation (all optional)
  uint8_t* C_scale = nullptr;      // fp6 output (tiled kernel): C is the packed operand [M, 3N/4], this its E8M0 bytes [M, N/32]
  int fmt_c = 0;                   // 2 / 3: format of the fp6 output; 0: bf16 / fp32 output
  int raster_group_m = 0, raster_no_xcd_remap = 0;  // tiled kernel, measurement only: tile rows per raster group (0 = the default, 4), XCD remap off (1), or on with a K split's workgroups in tile-by-tile order (2)
  int ablation = 0;  // tiled kernel, measurement only: leave out LDS reads (1), loads (2), MFMAs (4); results are then meaningless
  uint32_t* clock_stamps = nullptr;  // tiled kernel, measurement only: four words for workgroup 0's clock / real-time counters at start and end
  int no_alloc = 0;                // skinny kernel: the K split keeps its partial tiles in the library's static scratch array instead of an allocated workspace
  int force_split = 0;             // skinny kernel, M <= 32: split K between this many workgroups (1, 2, 4, 8); 0 = by shape
  int ksplit = 0;                  // tiled kernel: workgroups that share an output tile (from tiled_ksplit_plan, which also gives tile_rows); needs ks_part
  float* ks_part = nullptr;        // ... their partial sums: ksplit matrices [M, N] of floats (ring kernel: partial tiles)
  int* ks_counters = nullptr;      // ring kernel's K split: one arrival counter per tile of C, zero between launches
};

// the LDS-staged kernels fetch operands and scales 16 bytes per lane: all four tensors must be 16-byte aligned
inline bool operands_aligned16(const GemmArgs& g) {
  return (((uintptr_t)g.A | (uintptr_t)g.B | (uintptr_t)g.As | (uintptr_t)g.Bs) & 15) == 0;
}

// ---- kernel choice (dispatch.hip): candidates of the automatic path, a time model per candidate, a calibration table
enum Candidate : int { kCandTiled256 = 0, kCandTiled128x256, kCandTiled128x128, kCandBlock, kCandBlockWide, kCandSkinny, kCandTiledSplit256, kCandTiledSplit128, kCandBlockSplit, kCandRing, kNumCandidates };
struct KernelChoice {
  int cand;    // a Candidate, or -1: none of them takes the shape (the generic kernel does)
  int shares;  // K split: workgroups per output tile (1 = none)
  int rows;    // tiled kernel's split: rows of A per tile
  double us;   // modelled time x calibration factor
};
int device_cus();
double candidate_model_us(const GemmArgs& g, int cand, int want_split, int cus, int* shares, int* rows);  // modelled microseconds; < 0: the candidate does not take the shape
KernelChoice choose_kernel(const GemmArgs& g, int want_split, bool allow_split, unsigned mask = ~0u);  // mask: bit per Candidate that may be chosen; want_split: 0 = by the model, 1 = never, n = n shares where a candidate splits; allow_split: a workspace is to be had
int tiled_split_shares(const GemmArgs& g, int want, int cus, int bm);  // the tiled kernel's K split with tiles of bm (256 or 128) rows when it is to split: shares (1 = the shape has none)
int block_split_shares(const GemmArgs& g, int want, int cus);             // ... the block kernel's

hipError_t launch_gemm_generic(const GemmArgs& g, hipStream_t s);
bool gemm_tiled_supports(const GemmArgs& g);
hipError_t launch_gemm_tiled(const GemmArgs& g, hipStream_t s);
bool gemm_tiled4_supports(const GemmArgs& g);  // the 4-wave variant of the tiled kernel (selectable, never chosen automatically)
hipError_t launch_gemm_tiled4(const GemmArgs& g, hipStream_t s);
bool gemm_block_supports(const GemmArgs& g);  // 128 x 128 tiles, four waves in step (a few hundred to a few thousand rows of A)
hipError_t launch_gemm_block(const GemmArgs& g, hipStream_t s);
hipError_t launch_ksplit_reduce(const GemmArgs& g, hipStream_t s);  // sums g.ksplit partial matrices at g.ks_part into g.C, with the epilogue
bool gemm_ring_supports(const GemmArgs& g);  // batched decode: private streams of B per wave, A through a flag-guarded ring (no barrier per K-tile)
int ring_ksplit_plan(const GemmArgs& g, int want, size_t* part_bytes, size_t* counters);  // its K split for this problem (want: 0 = by shape, 1 = none, n = n shares): shares (1 = none), bytes of partial tiles, arrival counters
hipError_t launch_gemm_ring(const GemmArgs& g, hipStream_t s);
bool gemm_mid_supports(const GemmArgs& g);
hipError_t launch_gemm_mid(const GemmArgs& g, hipStream_t s);
bool gemm_skinny_supports(const GemmArgs& g);
hipError_t launch_gemm_skinny(const GemmArgs& g, hipStream_t s);
bool gemm_skinny_scratch_fits(const GemmArgs& g);  // no_alloc: the K split this call would use fits the static scratch array
hipError_t release_split_workspaces();             // returns every K-split workspace to the stream-ordered allocator
hipError_t launch_quantize(const void* X, int x_bf16, uint8_t* packed, uint8_t* scales, int rows, int K, int fmt, int layout, hipStream_t s);
hipError_t launch_tile_operand(const uint8_t* src, uint8_t* dst, int rows, int K, int tile, hipStream_t s);
hipError_t launch_tile_scales(const uint8_t* src, uint8_t* dst, int rows, int K, int tile, hipStream_t s);
hipError_t launch_tile_both(const uint8_t* src0, uint8_t* dst0, const uint8_t* ssrc0, uint8_t* sdst0, int rows0, const uint8_t* src1,
                            uint8_t* dst1, const uint8_t* ssrc1, uint8_t* sdst1, int rows1, int K, hipStream_t s);
hipError_t launch_fill_zero(void* p, size_t bytes, hipStream_t s);
hipError_t launch_mfma_probe(const uint8_t* A, const uint8_t* B, const uint8_t* As, const uint8_t* Bs, int rows_a, int rows_b, int K, int fmt_a,
                             int fmt_b, int iters, int workgroups, float* sink, uint32_t* stats, hipStream_t s);
hipError_t launch_stream_probe(const uint8_t* buf, size_t bytes, int workgroups, int waves, uint32_t* stats, hipStream_t s);

}  // namespace mxfp6
