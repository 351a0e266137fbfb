// LDS-tiled MXFP6 GEMM for gfx950: 256x256 output tile per workgroup, K-tile 128, 8 waves.
//
// Data path (no operand byte ever passes through a VGPR on its way to LDS):
//   global --buffer_load_dwordx4 ... lds--> LDS (3-stage ring) --ds_read_b128--> MFMA source VGPRs
//   v_mfma_scale_f32_32x32x64_f8f6f4 (fp32 accumulate, E8M0 block scales applied by the instruction)
//   accumulators --v_cvt_pk_bf16_f32, v_permlane32_swap--> 16 bytes per lane to global
// When there are more output tiles than compute units, one workgroup per CU walks through several tiles:
// the K-tiles of all its output tiles form one stream through the ring, so the loads of the next tile
// run under the last K-tiles of the current one and the stores of a finished tile under the first
// K-tiles of the next (measured: +1-2 % at K = 8192, +10 % at K = 1024; what remains per output tile,
// ~10 000 clocks at 8192^3, is the time all CUs together need to push 32 MB of C to HBM at once).
//
// LDS image of one operand tile (256 rows x 96 bytes = 6 pieces of 16 B per row): row-major, 96 bytes
// per row, with pieces 2p and 2p+1 exchanged in every row whose bit 3 is set:
//     piece c of row r lives at  r * 96 + (c ^ ((r >> 3) & 1)) * 16.
// A direct-to-LDS load writes lane l's 16 bytes at base + 16*l, so the image is produced by choosing
// which global bytes each lane fetches (the same idea as the reference's swizzled global offsets,
// include/ops/warp/memory/tile/global_to_shared.cuh:46-72).  Consecutive lanes fetch consecutive
// pieces of one row.  The pair exchange is what makes the reads conflict-free: a ds_read_b128
// executes in 16-lane phases ({0-3,12-15,20-23,24-27}, {4-11,16-19,28-31}, ... measured in
// analysis/paper_experiments/phases/ds_read_b128/phase_results.txt:4-7); with a 96-byte pitch rows r
// and r+8 would share banks, and every phase holds each (r mod 8) once with bit 3 clear and once set
// (measured here: 199 B/clk/CU with the exchange, 126 without).
// A tile-major operand (MXFP6_LAYOUT_TILE) is stored in global memory in exactly this order, which
// turns every load into one contiguous KiB; its scales are stored as the 512-byte chunks the scale
// loads fetch (32 rows x 16 bytes), 4 cache lines per 32 rows instead of 32.
//
// MFMA operand mapping: lane l of a 32x32x64 MFMA supplies row l%32 and one 32-element K-block.  Lanes
// 0-31 take K-blocks {0,1} of the K-tile and lanes 32-63 take K-blocks {2,3}: each lane reads its row's
// 48 contiguous bytes (three aligned 16-byte pieces) once and feeds two MFMAs (K-blocks {0,2} then {1,3}).
// Any assignment of K-blocks to lane halves is legal as long as both operands use the same one.
//
// E8M0 scales ride in LDS too: 16 bytes per row cover four K-tiles, fetched by one dwordx4 direct
// load per 64 rows per four K-tiles.  A lane needs bytes 2h and 2h+1 (h = lane / 32) of each K-tile's four: every
// second K-tile it reads the eight bytes of two K-tiles (ds_read_b64) and v_perm_b32 gathers its four into one
// register, of which the MFMAs' op_sel picks bytes 0, 1 (first K-tile of the pair) and 2, 3 (second).  (A
// ds_read_u16 per operand tile and K-tile, as before, was 30 % of all LDS cycles in bank conflicts and cost 16 %
// more shader clocks per GEMM.)
//
// Schedule: 8-wave ping-pong (the reference's pattern, analysis/bf16_gemm/mi325x/kernel_8192.cpp:75-153):
// waves 0-3 and waves 4-7 (one of each per SIMD) run half a K-tile out of phase, so that on every SIMD
// one wave issues MFMAs while the other reads LDS.  All waves are consumers (the reference measures
// all-consumer above producer/consumer, analysis/paper_experiments/producer_consumer_micro/plot.py:26-30).
// The direct loads are split between the two clusters: a load issued while four waves queue theirs at the
// same time stalls the wave for ~100 clocks (row-major operands; ~45 for contiguous ones), which is cheap
// between two MFMAs and expensive in front of the LDS reads, so kLoadsInCompute of a tile's six loads per
// wave ride in the compute cluster, one after every second MFMA, and the rest follow the LDS reads of the
// memory cluster (measured: memory cluster 1110 -> 720 clocks, 7 % / 11 % less time per GEMM for
// row-major / tile-major operands).
//
// This file is compiled five times (build.py): once as it is, which gives the host-side part (shape checks, tile
// shape and grid, the K split's reduction, the launcher that picks the format pair), and once per pair of operand
// formats with -DMXFP6_TILED_FMT=22 / 23 / 32 / 33, which gives that pair's kernel instantiations and launcher: the
// instantiations are what takes the time to compile, and four objects compile side by side.
#include "common.hpp"
#include "kernels.hpp"
#include "loader.hpp"

namespace mxfp6 {

// defined in the host-side object, used by the launchers of the per-format objects
int tiled_grid_size(const GemmArgs& g, int tiles, int per_cu);
hipError_t launch_ksplit_reduce(const GemmArgs& g, hipStream_t s);
constexpr int kMinShareTiles = 8;  // K-tiles a share of a K split has at least (dispatch.hip plans with the same figure)
// defined in the per-format objects
hipError_t launch_gemm_tiled_fmt22(const GemmArgs& g, hipStream_t s);
hipError_t launch_gemm_tiled_fmt23(const GemmArgs& g, hipStream_t s);
hipError_t launch_gemm_tiled_fmt32(const GemmArgs& g, hipStream_t s);
hipError_t launch_gemm_tiled_fmt33(const GemmArgs& g, hipStream_t s);

static constexpr int g_tiled_walk = 1;  // 0 would launch one workgroup per output tile everywhere (no walk)

constexpr int kBK = 128;  // the tile has 256 (TM = 4) or 128 (TM = 2) rows of A and 256 (TN = 2) or 128 (TN = 1) rows of B
constexpr int kGroupM = 4;          // tile rows per raster group
constexpr int WM = 2, WN = 4, NW = WM * WN;  // waves: 2 x 4, wave tile (TM * 32) x (TN * 32)
constexpr int SCL = 1;                       // scale direct loads per wave per slot that carries scales
// Per tile shape: TM (4 or 2) and TN (2 or 1) 32x32 MFMA tiles per wave in M and N.  A's tile of 128 rows against 256
// of B is 12 loads of 1 KB for 8 waves: waves 0-3 issue two each and waves 4-7 one (OPA1), so a batch is five loads for
// the first wave group and four for the second; the groups are instantiated separately anyway.  128 x 128 (SPLIT): both tiles are 12
// loads, waves 0-3 load A's and waves 4-7 B's, three each; no padding, and the scales take half the room (waves 2, 3,
// 6, 7 fetch the same 64 rows as waves 0, 1, 4, 5 again, into the same place, so that every wave issues the same number
// of loads): 80 KB, two workgroups per CU.
template <int TM, int TN>
struct Shape {
  static constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  static constexpr bool SPLIT = TM == 2 && TN == 1;
  static constexpr int OPA = SPLIT ? 3 : (BM * 96 / 1024 + NW - 1) / NW;  // direct loads per (loading) wave and K-tile for A (waves 0-3)
  static constexpr int OPA1 = SPLIT ? 3 : BM * 96 / 1024 / 4 - OPA;        // ... for waves 4-7: what is left of A's tile
  static constexpr int OPB = SPLIT ? 3 : (BN * 96 / 1024 + NW - 1) / NW;  // ... and for B
  static constexpr int NL = SPLIT ? 3 : OPA + OPB;                        // operand loads per wave and K-tile, waves 0-3
  static constexpr int NL1 = SPLIT ? 3 : OPA1 + OPB;                      // ... waves 4-7
  static_assert(SPLIT || (OPA1 >= 0 && 4 * (OPA + OPA1) * 1024 == BM * 96), "A's tile in whole loads");
  // of the operand loads per wave and K-tile: issued between MFMAs, one after every second of the 2 TM TN
  static constexpr int kLoadsInCompute = TM * TN < 4 ? TM * TN : 4;
  static constexpr int kAStage = BM * 96;                            // LDS bytes of A's tile
  static constexpr int kStage = kAStage + (SPLIT ? BN * 96 : OPB * NW * 1024);  // ... and of a ring slot
  static constexpr int kScStage = (SPLIT ? 128 : 256) * 16;  // bytes of one operand's scales for four K-tiles
  static constexpr int kScaleBuf = 2 * kScStage;
  // operand ring depth: three slots (two K-tiles in flight); four for the 128 x 256 tile, whose slots are 36 KB (three in
  // flight: that tile is used where few rows of A meet a wide B, and what bounds it there is how fast B streams from HBM)
  static constexpr int kStages = TM == 2 && TN == 2 ? 4 : 3;
  static constexpr int kScaleBase = kStages * kStage, kLdsBytes = kScaleBase + 2 * kScaleBuf;
  static_assert(kLoadsInCompute >= 0 && kLoadsInCompute <= NL && kLoadsInCompute <= NL1 && 2 * kLoadsInCompute <= 2 * TM * TN, "load slots");
  static_assert(kLdsBytes <= 163840, "LDS budget");
};

// (dma16, wait_vmcnt, wait_lds_reads, barrier: loader.hpp.  The ring keeps two K-tiles in flight across barriers, which
// the compiler's automatic waits would serialise: hence the loads from inline assembly and the VMEM counter by hand.)

// The kernel's arguments, passed as one struct: a workgroup that walks through several output tiles reads
// them again from the kernel-argument segment whenever it moves on, instead of keeping all of them in
// scalar registers through the K loop.
struct TiledArgs {
  const uint8_t *A, *B, *As, *Bs;
  void* C;
  int M, N, K, tiles_m, tiles_n, layout_a, layout_b;
  Epilogue ep;
  uint8_t* C_scale;  // fp6 output only
  int fmt_c;
  int group_m, xcd_remap;  // raster: tile rows per group (kGroupM unless a measurement overrides it), XCD remap on / off
  int nsplit;        // KSPLIT: workgroups that share an output tile, each over K / nsplit (1 otherwise)
#ifdef MXFP6_PROBES
  uint32_t* stamps;  // measurement build only (else null): workgroup 0 leaves its shader-clock and real-time counters here at start and end
#endif
};

// FUSED: the epilogue applies scales / bias / activation (args.ep).  A separate instantiation, because branches
// around updates of all accumulators make the compiler copy them at every output tile, taken or not (3-4 % of an
// unfused 8192^3 GEMM).
// ABL (measurement build only, -DMXFP6_PROBES; results are then meaningless): bit 0 leaves out the LDS reads of the operands after the first
// K-tile of an output tile, bit 1 the direct loads after the prologue, bit 2 the MFMAs after the first K-tile of an output
// tile; bit 3 leaves everything in and adds idle clocks (a wave sleeps 128 clocks after every fourth MFMA).  What the remaining parts of the kernel take, in time and in shader clocks, is how bench.py splits the kernel's
// time between the matrix cores, the LDS reads and the loads.
// KSPLIT: the K range of an output tile is split between args.nsplit workgroups (few output tiles, long K: M of a few
// hundred rows).  Share s of a tile multiplies K-tiles [s, s + 1) * nkt / nsplit and stores its fp32 sums into matrix s of
// args.C, which is then a workspace of nsplit matrices [M, N]; ksplit_reduce_kernel adds them in share order and applies
// the epilogue.  (Summed inside this kernel instead -- partial tiles and arrival counters at device scope, the last
// wave to arrive adds -- the few waves that end up adding read nsplit tiles each past the L2s: 30 us for 32 MB.)
template <int FA, int FB, typename Out, int TM, int TN, bool FUSED, int ABL = 0, bool KSPLIT = false>
__global__ __launch_bounds__(NW * 64) void gemm_tiled_kernel(const TiledArgs args) {
  typedef Shape<TM, TN> S;
  constexpr int kBM = S::BM, kBN = S::BN, OPA = S::OPA, OPA1 = S::OPA1, OPB = S::OPB, kLoadsInCompute = S::kLoadsInCompute;
  constexpr int kAStage = S::kAStage, kStage = S::kStage, kScaleBase = S::kScaleBase, kScStage = S::kScStage, kScaleBuf = S::kScaleBuf;
  constexpr int kStages = S::kStages, D = kStages - 1;  // D: how many K-tiles ahead of the one being multiplied the loads run
  constexpr bool SPLIT = S::SPLIT;
  static_assert(TN == 2 || sizeof(typename Out::type) != 1, "the fp6 epilogue pairs a wave's two tiles of a band");
  // LDS map: [stage 0..2][A tile | B tile] then [scale buffer 0..1][A scales | B scales]
  __shared__ __attribute__((aligned(1024))) uint8_t smem[S::kLdsBytes];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem;
  const int K = args.K, layout_a = args.layout_a, layout_b = args.layout_b;
  const int rowbytes = K / 4 * 3, sbytes = K / 32, nkt_all = K / kBK;
  const int nk4_all = (nkt_all + 3) / 4;  // groups of four K-tiles; tile-major scales hold one 512-byte chunk per 32 rows and group
  // K-tiles (and groups of four) of one workgroup's share of an output tile: all of them, or (KSPLIT) a whole number of groups
  const int nkt = KSPLIT ? nkt_all / args.nsplit : nkt_all, nk4 = KSPLIT ? nkt / 4 : nk4_all;
  static_assert(!KSPLIT || (!Shape<TM, TN>::SPLIT && sizeof(typename Out::type) == 4 && ABL == 0 && !FUSED), "K split: 256 rows of B, plain fp32 partial sums");
  const bool sc_a = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) < 4;  // this wave loads A's scales (else B's)

  // the arguments, read afresh (the empty asm hides from the compiler that the pointer is always the same)
  auto fresh_args = [&]() __attribute__((always_inline)) {
    auto p = (const __attribute__((address_space(4))) TiledArgs*)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));
    return p;
  };

  // ---- workgroup -> output tiles: workgroup b works on tiles b, b + gridDim.x, ... of tile_order() (common.hpp)
  // KSPLIT: workgroup b takes share l / tiles of tile l % tiles, l = ksplit_order(b): share-major, an eighth of it per XCD
  auto split_order_of = [&](int bid) __attribute__((always_inline)) {  // bid < tiles * nsplit
    const auto g = fresh_args();
    return ksplit_order(bid, g->tiles_m * g->tiles_n * g->nsplit, g->xcd_remap);
  };
  auto tile_of = [&](int bid) __attribute__((always_inline)) {
    const auto g = fresh_args();
    if constexpr (KSPLIT) {
      const int tiles = g->tiles_m * g->tiles_n, total = tiles * g->nsplit;
      if (bid >= total) return -1;
      const bool by_share = ksplit_by_share(total, g->xcd_remap);  // the XCDs are dealt by ksplit_order, not by tile_order
      return tile_order(split_order_of(bid) % tiles, g->tiles_m, g->tiles_n, g->group_m, by_share ? 0 : g->xcd_remap);
    }
    return tile_order(bid, g->tiles_m, g->tiles_n, g->group_m, g->xcd_remap);
  };
  // share of workgroup bid (a workgroup with a tile: bid < tiles * nsplit); 0 without the split
  auto share_of = [&](int bid) __attribute__((always_inline)) {
    if constexpr (KSPLIT) {
      const auto g = fresh_args();
      const int tiles = g->tiles_m * g->tiles_n;
      return bid < tiles * g->nsplit ? split_order_of(bid) / tiles : 0;
    }
    return 0;
  };
  // first K-tile of workgroup-share bid (0 without the split)
  auto ktile0_of = [&](int bid) __attribute__((always_inline)) { return share_of(bid) * nkt; };
  // Buffer resources of one output tile's operand rows (A and B) and of the scale rows this wave loads.  Edge
  // tiles: rows past M (or N) lie beyond the end of the resource and read as zeros.  tile < 0: resources of
  // length zero, loads through them fetch nothing.
  __amdgpu_buffer_rsrc_t rA, rB, rS;
  // kt0 (KSPLIT): the share's first K-tile; the resources start there (K-tile kt0 of a row or row-tile is 96 or 3072 bytes
  // times kt0 into it) and end that much earlier, so that rows past the tile's last still lie beyond the end.
  auto operand_rsrc = [&](int tile, int kt0) __attribute__((always_inline)) {
    const auto g = fresh_args();
    const int pm = tile < 0 ? 0 : tile & 0xffff, pn = tile < 0 ? 0 : tile >> 16;
    const int rows_a = tile < 0 ? 0 : min(kBM, g->M - pm * kBM), rows_b = tile < 0 ? 0 : min(kBN, g->N - pn * kBN);
    if constexpr (SPLIT) {  // a wave loads one operand only: rA is that operand's resource (no branch at the loads)
      rA = sc_a ? make_rsrc(g->A + (size_t)pm * kBM * rowbytes, (uint32_t)rows_a * rowbytes)
                : make_rsrc(g->B + (size_t)pn * kBN * rowbytes, (uint32_t)rows_b * rowbytes);
    } else if constexpr (KSPLIT) {
      const uint32_t oa = tile < 0 ? 0 : (uint32_t)kt0 * (layout_a ? 3072 : 96), ob = tile < 0 ? 0 : (uint32_t)kt0 * (layout_b ? 3072 : 96);
      rA = make_rsrc(g->A + (size_t)pm * kBM * rowbytes + oa, (uint32_t)rows_a * rowbytes - oa);
      rB = make_rsrc(g->B + (size_t)pn * kBN * rowbytes + ob, (uint32_t)rows_b * rowbytes - ob);
    } else {
      rA = make_rsrc(g->A + (size_t)pm * kBM * rowbytes, (uint32_t)rows_a * rowbytes);
      rB = make_rsrc(g->B + (size_t)pn * kBN * rowbytes, (uint32_t)rows_b * rowbytes);
    }
  };
  auto scale_rsrc = [&](int tile, int kt0) __attribute__((always_inline)) {
    const auto g = fresh_args();
    const int pm = tile < 0 ? 0 : tile & 0xffff, pn = tile < 0 ? 0 : tile >> 16;
    const int rows_a = tile < 0 ? 0 : min(kBM, g->M - pm * kBM), rows_b = tile < 0 ? 0 : min(kBN, g->N - pn * kBN);
    const uint8_t* sp = sc_a ? g->As : g->Bs;
    const int slay = sc_a ? layout_a : layout_b, srows = sc_a ? rows_a : rows_b, stile = sc_a ? pm : pn;
    const int sheight = sc_a ? kBM : kBN;  // rows per tile of the operand whose scales these are
    const uint32_t off = KSPLIT && tile >= 0 ? (uint32_t)(kt0 >> 2) * (slay ? 512 : 16) : 0;  // the share's first group of four K-tiles
    rS = slay ? make_rsrc(sp + (size_t)stile * (sheight / 32) * nk4_all * 512 + off, (uint32_t)((srows + 31) / 32) * nk4_all * 512 - off)
              : make_rsrc(sp + (size_t)stile * sheight * sbytes + off, (uint32_t)srows * sbytes - off);
  };
  int bid_cur = blockIdx.x, bid_next = blockIdx.x + gridDim.x;
  int tile_cur = tile_of(bid_cur), tile_next = tile_of(bid_next);
  operand_rsrc(tile_cur, ktile0_of(bid_cur));
  scale_rsrc(tile_cur, ktile0_of(bid_cur));

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int h = lane >> 5, r32 = lane & 31;

  // per-lane global byte offsets of the direct loads.  Load q = wave*OPA + i (A) or wave*OPB + i (B) fills
  // LDS bytes [q*1024, q*1024 + 1024) of the operand tile.  Row-major operand: slot o holds piece
  // (o%6) ^ ((row>>3)&1) of row o/6, K-tile t starts at byte 96 t of a row.  Tile-major operand:
  // the 3072-byte tile of 32 rows is stored in exactly this order, so the load is one contiguous
  // KiB, row-tiles are (K/128)*3072 bytes apart and K-tile t starts at byte 3072 t.
  int voff_a[OPA], voff_b[OPB];
  auto load_offset = [&](int q, int layout) __attribute__((always_inline)) {
    const int o = q * 64 + lane;  // linear 16-byte slot inside the LDS image
    const int r = o / 6, c = (o - r * 6) ^ ((r >> 3) & 1);
    const int vrow = r * rowbytes + c * 16;
    const int vtile = (q / 3) * (nkt_all * 3072) + (q % 3) * 1024 + lane * 16;
    return layout ? vtile : vrow;
  };
  const int qa0 = wave < 4 ? wave * OPA : 4 * OPA + (wave - 4) * OPA1;  // this wave's first load of A's tile (waves 4-7 issue OPA1 of them)
#pragma unroll
  for (int i = 0; i < OPA; i++) voff_a[i] = SPLIT ? load_offset((wave & 3) * OPA + i, sc_a ? layout_a : layout_b) : load_offset(qa0 + i, layout_a);
#pragma unroll
  for (int i = 0; i < OPB; i++) voff_b[i] = SPLIT ? 0 : load_offset(wave * OPB + i, layout_b);
  const int kstep_a = (SPLIT && !sc_a ? layout_b : layout_a) ? 3072 : 96, kstep_b = layout_b ? 3072 : 96;
  const int split_base = (sc_a ? 0 : kAStage) + (wave & 3) * (OPA * 1024);  // SPLIT: where this wave's three loads land in a ring slot
  // scales: a lane fetches the 16 scale bytes (four K-tiles) of one row; waves 0-3 load A's, 4-7 B's
  const int swave = SPLIT ? wave & 1 : wave & 3;  // which 64 rows of the operand's tile this wave fetches the scales of
  const int srow = swave * 64 + lane, slay = wave < 4 ? layout_a : layout_b;
  const int voff_s = slay ? (srow >> 5) * nk4_all * 512 + (srow & 31) * 16 : srow * sbytes;
  const int sstep = slay ? 512 : 16;  // bytes between consecutive groups of four K-tiles

  // per-lane LDS read offsets (bytes from the start of a stage): the lane's three pieces 3h..3h+2
  const int sw = (r32 >> 3) & 1;
  int a_rd[3], b_rd[3];
#pragma unroll
  for (int c = 0; c < 3; c++) {
    a_rd[c] = (wm * (TM * 32) + r32) * 96 + ((3 * h + c) ^ sw) * 16;
    b_rd[c] = kAStage + (wn * (TN * 32) + r32) * 96 + ((3 * h + c) ^ sw) * 16;
  }
  const int sa_rd = kScaleBase + (wm * (TM * 32) + r32) * 16;
  const int sb_rd = kScaleBase + kScStage + (wn * (TN * 32) + r32) * 16;

  v16f acc[TM][TN];  // never zeroed: the first K-tile of an output tile multiplies into a zero C operand

  int p0 = 0;  // scale buffer that holds group 0 of the current output tile

  // ---- loads.  A wave's batch for K-tile t is its NL (waves 4-7: NL1) operand loads (n = 0..OPA-1: A, then B) and,
  // when t % 4 == 2, the scale load for the four K-tiles starting at t + 2 (at the end of the batch, so
  // that a wait that leaves a whole batch in flight also covers the scales of the batch before).
  // K-tile (or group of four K-tiles) number kk counts on from the current output tile into the next one.
  // The resources rA, rB (and rS) are those of the output tile the loads have reached: they move on to the
  // next output tile just before the first load that belongs to it, and past the workgroup's last output
  // tile to empty resources.  INSIDE says that the caller knows kk to lie in the current tile.
  [[maybe_unused]] bool abl_started = false;  // ABL & 2: the prologue is over
  auto issue_scales = [&]<bool INSIDE>(int grp) __attribute__((always_inline)) {
    if constexpr ((ABL & 2) != 0) {
      if (abl_started) return;
    }
    const int buf = (p0 + grp) & 1;
    const uint32_t dst = lds0 + kScaleBase + buf * kScaleBuf + swave * 1024;
    // the group's offset rides in the per-lane offset, which the hardware checks against the end of the resource (the
    // scalar offset it does not): with K % 512 != 0 the last group of a row-major row is shorter than 16 bytes, and the
    // last row's load must not read past the tensor
    dma16(rS, sc_a ? dst : dst + kScStage, voff_s + (INSIDE || grp < nk4 ? grp : grp - nk4) * sstep, 0);
  };
  auto issue_one = [&]<bool INSIDE, int GRP>(int kk, int slot, int n) __attribute__((always_inline)) {
    constexpr int OPAg = GRP == 0 ? OPA : OPA1;
    if constexpr ((ABL & 2) != 0) {
      if (abl_started) return;
    }
    const int t = INSIDE || kk < nkt ? kk : kk - nkt;
    const uint32_t dst = lds0 + slot * kStage;
    if constexpr (SPLIT) {
      dma16(rA, dst + split_base + n * 1024, voff_a[n], t * kstep_a);
    } else {
      if (n < OPAg) dma16(rA, dst + (qa0 + n) * 1024, voff_a[n], t * kstep_a);
      else dma16(rB, dst + kAStage + (wave * OPB + n - OPAg) * 1024, voff_b[n - OPAg], t * kstep_b);
    }
  };

  // ---- one K-tile: LDS -> registers (memory cluster) and the MFMAs (compute cluster)
  // a lane's 48 bytes of one 32-row tile live in 12 consecutive VGPRs: dwords 0-5 are the operand of the
  // first MFMA, 6-11 of the second
  v12i fa[TM], fb[TN];
  int sca[TM], scb[TN];  // this lane's scale bytes of a pair of K-tiles: bytes 0, 1 the first K-tile's two blocks, 2, 3 the second's
  // KM: K-tile modulo 4.  sc_off: the scale buffer of the K-tile's group of four.
  auto read_tile = [&]<int KM>(int stage, int sc_off) __attribute__((always_inline)) {
    const uint8_t* st = smem + stage * kStage;
    const uint8_t* sc = smem + sc_off + (KM >> 1) * 8;
    // byte selector of v_perm_b32 for this lane's half, recomputed here instead of living in a register through the loop
    uint32_t sc_sel = 0;
    if ((KM & 1) == 0) {
      int lid = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
      asm volatile("" : "+v"(lid));
      sc_sel = lid & 32 ? 0x07060302u : 0x05040100u;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const v4i p = *reinterpret_cast<const v4i*>(st + b_rd[c] + j * 3072);
#pragma unroll
        for (int e = 0; e < 4; e++) fb[j][4 * c + e] = p[e];
      }
      if ((KM & 1) == 0) {
        const v2i raw = *reinterpret_cast<const v2i*>(sc + sb_rd + j * 512);
        scb[j] = __builtin_amdgcn_perm(raw[1], raw[0], sc_sel);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const v4i p = *reinterpret_cast<const v4i*>(st + a_rd[c] + i * 3072);
#pragma unroll
        for (int e = 0; e < 4; e++) fa[i][4 * c + e] = p[e];
      }
      if ((KM & 1) == 0) {
        const v2i raw = *reinterpret_cast<const v2i*>(sc + sa_rd + i * 512);
        sca[i] = __builtin_amdgcn_perm(raw[1], raw[0], sc_sel);
      }
    }
  };
  // first K-block of every lane for all tiles, then the second: two MFMAs into the same accumulator
  // are TM*TN instructions apart.  First source = B rows (index n), second = A rows (index m): a lane
  // ends up owning 4 consecutive n of row m = lane % 32, four times.  FIRST: the K-tile opens an output tile,
  // so the first MFMA into every accumulator takes zero as its C operand.  between(i) runs after the i-th MFMA.
  auto mma_tile = [&]<bool FIRST, int KM>(auto&& between) __attribute__((always_inline)) {
    constexpr int S0 = 2 * (KM & 1), S1 = S0 + 1;  // op_sel: which byte of the scale registers
    if ((ABL & 4) && !FIRST) {
#pragma unroll
      for (int q = 0; q < 2 * TM * TN; q++) between(q);
      return;
    }
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const v8i a0 = __builtin_shufflevector(fa[i], fa[i], 0, 1, 2, 3, 4, 5, -1, -1);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const v8i b0 = __builtin_shufflevector(fb[j], fb[j], 0, 1, 2, 3, 4, 5, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, S0, S0>(b0, a0, FIRST ? zero : acc[i][j], scb[j], sca[i]);
        between(i * TN + j);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const v8i a1 = __builtin_shufflevector(fa[i], fa[i], 6, 7, 8, 9, 10, 11, -1, -1);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const v8i b1 = __builtin_shufflevector(fb[j], fb[j], 6, 7, 8, 9, 10, 11, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, S1, S1>(b1, a1, acc[i][j], scb[j], sca[i]);
        between(TM * TN + i * TN + j);
      }
    }
  };

  // ---- the K loop.  Barrier n is common to all waves; between barriers 2k and 2k+1 group 0 (waves
  // 0-3) is in its memory cluster for tile k and between 2k+1 and 2k+2 in its compute cluster; group 1
  // (waves 4-7) does the same one barrier later.  A ring slot is refilled only after the barrier by
  // which both groups have finished reading it, and each wave waits for its own share of tile k+1
  // before the barrier that precedes the first read of that tile.
  // Loads of step k, with D = ring slots - 1 (2, or 3 for the 128 x 256 tile).  Memory cluster, after the LDS reads, both
  // groups: loads kLoadsInCompute.. of tile k+D (slot of tile k-1, free since barrier 2k) and the scales.  Compute
  // cluster: loads 0..kLoadsInCompute-1, for group 0 of the same tile k+D, for group 1 of tile k+D+1, whose slot is the
  // one of tile k: group 1's compute cluster starts at barrier 2k+2, by which both groups have read
  // tile k.  In program order every tile's batch is contiguous for both groups, so one wait count
  // serves both: everything older than the D - 1 newest batches has landed.
  // The K-tiles of all output tiles of a workgroup form ONE stream: K-tile k+D or k+D+1 past the end of
  // an output tile is one of the first K-tiles of the workgroup's next output tile, so the ring never drains
  // between output tiles, and the finished tile's stores run while the other group still multiplies.
  // Past the last output tile the stream continues with loads through an empty buffer resource: they
  // fetch nothing and fill ring slots nobody reads, which keeps every step's load and wait pattern the same.
  // The body is instantiated per group (GRP) and per k mod 4 (KM); STEADY means that tiles k+D, k+D+1 and
  // (for the scales) k+4 lie in the current output tile, so its loads need no choice of descriptor.
  int stage = 0, stage2 = D;  // ring slots of tile k and tile k+D
  auto step = [&]<int GRP, int KM, bool STEADY, bool FIRST>(int kt) __attribute__((always_inline)) {
    constexpr int AHEAD = GRP == 0 ? D : D + 1;
    constexpr int NL = GRP == 0 ? S::NL : S::NL1;
    // loads left in flight by this step's wait: the D - 1 newest batches (K-tiles k+2 .. k+D), and the scale loads among
    // them (the batch of K-tile k+j was issued in step k+j-D and carries one if that step's k mod 4 is 0)
    constexpr int kInFlight = (D - 1) * NL + SCL * (((KM + 2 - D + 4) % 4 == 0) + (D == 3 && KM == 0));
    // outside the steady state every step derives its offsets and choices from kt on the spot: related to each
    // other across the steps of a trip they become a few dozen induction variables in scalar registers
    if (!STEADY) asm volatile("" : "+s"(kt));
    const int slotx = GRP == 0 ? stage2 : stage;
    if (!(ABL & 1) || FIRST) read_tile.template operator()<KM>(stage, ((p0 + (kt >> 2)) & 1) * kScaleBuf);
    __builtin_amdgcn_sched_barrier(0);
    // the loads reach the next output tile: group 0's with K-tile kt+2 at the start of a step, group 1's
    // with K-tile kt+3 in its compute cluster; the scales with group nk4
    if (!STEADY && GRP == 0 && kt + D == nkt) operand_rsrc(tile_next, ktile0_of(bid_next));
#pragma unroll
    for (int n = kLoadsInCompute; n < NL; n++) issue_one.template operator()<STEADY, GRP>(kt + D, stage2, n);
    if (KM == 0) {
      if (!STEADY && (kt + 4) >> 2 == nk4) scale_rsrc(tile_next, ktile0_of(bid_next));
      issue_scales.template operator()<STEADY>((kt + 4) >> 2);
    }
    if (!STEADY && GRP == 1 && kt + D + 1 == nkt) operand_rsrc(tile_next, ktile0_of(bid_next));
    wait_lds_reads();  // this tile's LDS reads are done before anyone may refill its slot
    // the middle 16-byte piece straddles the two operands; naming each fragment as one 384-bit value here
    // makes the register allocator keep it in one tuple, and the MFMAs read sub-tuples of it instead of
    // copies (24 v_mov per K-tile otherwise)
#pragma unroll
    for (int i = 0; i < TM; i++) asm volatile("" : "+v"(fa[i]));
#pragma unroll
    for (int j = 0; j < TN; j++) asm volatile("" : "+v"(fb[j]));
    // own share of the next K-tile has landed; the batch after it may be in flight
    if (GRP == 1) wait_vmcnt<kInFlight>();
    barrier();
    __builtin_amdgcn_s_setprio(1);
    mma_tile.template operator()<FIRST, KM>([&](int i) __attribute__((always_inline)) {
      if ((i & 1) && i / 2 < kLoadsInCompute) {
        __builtin_amdgcn_sched_barrier(0);
        issue_one.template operator()<STEADY, GRP>(kt + AHEAD, slotx, i / 2);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr ((ABL & 8) != 0) {  // the full kernel with idle clocks added: the wave sleeps 128 clocks after every fourth MFMA
        if ((i & 3) == 3) {
          __builtin_amdgcn_sched_barrier(0);
          __builtin_amdgcn_s_sleep(2);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    });
    __builtin_amdgcn_s_setprio(0);
    if (GRP == 0) wait_vmcnt<kInFlight>();
    barrier();
    stage = stage == kStages - 1 ? 0 : stage + 1;
    stage2 = stage2 == kStages - 1 ? 0 : stage2 + 1;
  };
  auto k_loop = [&]<int GRP>() __attribute__((always_inline)) {
    // first four K-tiles of the output tile (the first of them starts the accumulators)
    if (nkt >= 8) {
      step.template operator()<GRP, 0, true, true>(0);
      step.template operator()<GRP, 1, true, false>(1);
      step.template operator()<GRP, 2, true, false>(2);
      step.template operator()<GRP, 3, true, false>(3);
    } else {
      step.template operator()<GRP, 0, false, true>(0);
      if (1 < nkt) step.template operator()<GRP, 1, false, false>(1);
      if (2 < nkt) step.template operator()<GRP, 2, false, false>(2);
      if (3 < nkt) step.template operator()<GRP, 3, false, false>(3);
    }
    int kt = 4;
    for (; kt + 8 <= nkt; kt += 4) {  // four tiles per trip, all of them with tiles kt+2 .. kt+7 in range
      step.template operator()<GRP, 0, true, false>(kt);
      step.template operator()<GRP, 1, true, false>(kt + 1);
      step.template operator()<GRP, 2, true, false>(kt + 2);
      step.template operator()<GRP, 3, true, false>(kt + 3);
    }
    for (; kt < nkt; kt += 4) {  // last (up to seven) tiles: same body with the range checks
      step.template operator()<GRP, 0, false, false>(kt);
      if (kt + 1 < nkt) step.template operator()<GRP, 1, false, false>(kt + 1);
      if (kt + 2 < nkt) step.template operator()<GRP, 2, false, false>(kt + 2);
      if (kt + 3 < nkt) step.template operator()<GRP, 3, false, false>(kt + 3);
    }
  };

  // ---- epilogue of one output tile, straight from the accumulators.  Register v of lane l is C[m][n] with
  // m = l % 32 and n = 8 (v / 4) + 4 (l / 32) + v % 4 inside every 32x32 tile: lanes l and l + 32 hold the two
  // halves of each run of 8 consecutive n of one row.  bf16: after the conversion the two lanes trade halves
  // (v_permlane32_swap: the upper lanes' first run for the lower lanes' second), so that every lane owns 8
  // consecutive outputs and stores them as 16 bytes; two stores complete a row's 64-byte sector and four its
  // 128-byte line, back to back.  (8 bytes per lane and row, the accumulators as they are, measured 1.4x the
  // output in HBM write traffic; 4 bytes per lane with rows down the lanes, 64 stores per wave, measured
  // ~47 clocks per store instruction.)  Nothing here touches LDS, so the ring keeps streaming the next output
  // tile meanwhile.  The stores count in vmcnt like the loads and retire in order with them, so the waits of
  // the K loop ("all but the newest batch") stay valid.
  // EDGE: the tile has fewer than 256 valid rows or columns; those stores are predicated per lane.
  typedef typename Out::type OutT;
  // Fused scales / bias / activation, on the accumulators themselves, before the epilogue proper.  Per 32x32 tile a
  // lane owns row wm * TM * 32 + 32 i + lane % 32 and columns 8 q + 4 h .. + 3 for q = 0..3; N % 8 == 0, so a run of
  // four is inside or outside N as a whole.  The loads here are the compiler's: its waits also wait for the direct
  // loads in flight, which costs a fused call a fraction of a K-tile per output tile and an unfused one nothing.
  auto fuse = [&]() __attribute__((always_inline)) {
    const auto g = fresh_args();
    const void* bias = g->ep.bias;
    const float *row_scale = g->ep.row_scale, *col_scale = g->ep.col_scale;
    const int act = g->ep.act, bias_bf16 = g->ep.bias_bf16;
    const bool affine = bias || row_scale || col_scale;
    const int M = g->M, N = g->N;
    const long m0 = (long)(tile_cur & 0xffff) * kBM + wm * (TM * 32) + r32, n0 = (long)(tile_cur >> 16) * kBN + wn * (TN * 32) + 4 * h;
    // 32 columns (j) at a time, each with its own branches: a branch around all 128 accumulators at once makes the
    // compiler keep a second copy of them.  The column vectors of a j are loaded once for all rows (one round of load
    // latency per j and output tile, not per 32x32 tile).
    float rs[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) rs[i] = row_scale && m0 + i * 32 < M ? row_scale[m0 + i * 32] : 1.f;
#pragma unroll
    for (int j = 0; j < TN; j++) {
      if (affine) {
        v4f cs[4], bi[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const long n = n0 + j * 32 + q * 8;
          cs[q] = v4f{1.f, 1.f, 1.f, 1.f}, bi[q] = v4f{0.f, 0.f, 0.f, 0.f};
          if (n < N) {
            if (col_scale) cs[q] = *reinterpret_cast<const v4f*>(col_scale + n);
            if (bias && bias_bf16) {
              const u32x2 b2 = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(bias) + n);
              bi[q] = v4f{__uint_as_float(b2[0] << 16), __uint_as_float(b2[0] & 0xffff0000u), __uint_as_float(b2[1] << 16),
                          __uint_as_float(b2[1] & 0xffff0000u)};
            } else if (bias) {
              bi[q] = *reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(bias) + n);
            }
          }
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int q = 0; q < 4; q++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][4 * q + e] = fmaf(acc[i][j][4 * q + e] * rs[i], cs[q][e], bi[q][e]);
      }
#pragma unroll
      for (int i = 0; i < TM; i++) {
        if (act == 1) {
#pragma unroll
          for (int e = 0; e < 16; e++) acc[i][j][e] = act_relu(acc[i][j][e]);
        } else if (act == 2) {
#pragma unroll
          for (int e = 0; e < 16; e++) acc[i][j][e] = act_gelu(acc[i][j][e]);
        } else if (act == 3) {
#pragma unroll
          for (int e = 0; e < 16; e++) acc[i][j][e] = act_silu(acc[i][j][e]);
        }
        asm volatile("" : "+v"(acc[i][j]));
      }
    }
  };
  auto epilogue = [&]<bool EDGE>(int rows_a, int rows_b) __attribute__((always_inline)) {
    const auto g = fresh_args();
    if constexpr (sizeof(OutT) == 1) {
      // C re-quantised to MXFP6 along N (the next GEMM's K): a 32-block of row m is the 16 values of lane (m, h = 0)
      // and the 16 of lane (m, h = 1) of one 32x32 tile.  The wave's two tiles of a band (j = 0, 1) are traded with
      // v_permlane32_swap, register by register, after which the lower lane holds all of block j = 0 and the upper
      // lane all of block j = 1: P0[k] = column 8 (k / 4) + k % 4, P1[k] = that + 4.  Then exactly the quantiser:
      // amax -> E8M0 -> hardware conversion -> 24 bytes and a scale byte per lane.
      const int N = g->N, nkb = N / 32, fmt_c = g->fmt_c;
      const long m0 = (long)(tile_cur & 0xffff) * kBM + wm * (TM * 32) + r32;
      const int blk = (tile_cur >> 16) * (kBN / 32) + wn * TN + h;  // 32-block index along N of this lane's block
      uint8_t* cp = reinterpret_cast<uint8_t*>(g->C);
      uint8_t* sp = g->C_scale;
      const int M = g->M;
#pragma unroll
      for (int i = 0; i < TM; i++) {
        float p0[16], p1[16];
#pragma unroll
        for (int k = 0; k < 16; k++) {
          const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[i][0][k]), __float_as_uint(acc[i][1][k]), false, false);
          p0[k] = __uint_as_float(sw[0]), p1[k] = __uint_as_float(sw[1]);
        }
        float amax = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) amax = fmaxf(amax, fmaxf(fabsf(p0[k]), fabsf(p1[k])));
        const int sb = e8m0_of_amax(amax, fmt_c == 2 ? 2 : 4);
        const float scale = __uint_as_float((uint32_t)sb << 23);
        v16f ev, od;  // even and odd columns of the block: column n = 8 q + r is p0[4 q + r] for r < 4, p1[4 q + r - 4] otherwise
#pragma unroll
        for (int t = 0; t < 16; t++) {
          const int ne = 2 * t, no = 2 * t + 1;
          ev[t] = (ne & 4) ? p1[4 * (ne >> 3) + (ne & 3)] : p0[4 * (ne >> 3) + (ne & 3)];
          od[t] = (no & 4) ? p1[4 * (no >> 3) + (no & 3)] : p0[4 * (no >> 3) + (no & 3)];
        }
        typedef unsigned v6u __attribute__((ext_vector_type(6)));
        // a real branch (the empty asm keeps it one): with both conversions issued on the same sources and a select
        // behind them, the second one's result came out wrong from the third dword on
        v6u w;
        if (fmt_c == 2) {
          w = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(ev, od, scale);
          asm volatile("" : "+v"(w));
        } else {
          w = __builtin_amdgcn_cvt_scalef32_2xpk16_bf6_f32(ev, od, scale);
          asm volatile("" : "+v"(w));
        }
        const long m = m0 + i * 32;
        if (m < M && blk < nkb) {
          u32x2* dst = reinterpret_cast<u32x2*>(cp + (m * nkb + blk) * 24);
#pragma unroll
          for (int c = 0; c < 3; c++) dst[c] = u32x2{w[2 * c], w[2 * c + 1]};
          sp[m * nkb + blk] = (uint8_t)sb;
        }
      }
      return;
    }
    const int N = g->N, N2 = N * (int)sizeof(OutT);  // N2: bytes per row of C
    // the resource ends with the tile's last valid element
    OutT* cbase = (OutT*)g->C;
    if constexpr (KSPLIT) cbase += (size_t)share_of(bid_cur) * g->M * N;  // this share's matrix
    const __amdgpu_buffer_rsrc_t rC = make_rsrc(cbase + (size_t)(tile_cur & 0xffff) * kBM * N + (size_t)(tile_cur >> 16) * kBN,
                                                (uint32_t)((rows_a - 1) * N + rows_b) * (uint32_t)sizeof(OutT));
    const int row_l = wm * (TM * 32) + r32;
    if constexpr (sizeof(OutT) == 2) {
      const int col_l = wn * (TN * 32) + 8 * h;
      const int voff = row_l * N2 + col_l * 2;
#pragma unroll
      for (int i = 0; i < TM; i++) {
        // each phase for the whole 32-row band before the next one, so that no dword waits for its predecessor
        uint32_t pk[TN][8];
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int e = 0; e < 8; e++) pk[j][e] = pack_bf16x2(acc[i][j][2 * e], acc[i][j][2 * e + 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int t = 0; t < 2; t++)
#pragma unroll
            for (int c = 0; c < 2; c++) {
              // runs 2t and 2t+1 (dwords 4t+c and 4t+2+c): lower lanes keep run 2t and get the partner's, upper lanes run 2t+1
              const auto sw = __builtin_amdgcn_permlane32_swap(pk[j][4 * t + c], pk[j][4 * t + 2 + c], false, false);
              pk[j][4 * t + c] = sw[0], pk[j][4 * t + 2 + c] = sw[1];
            }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int t = 0; t < 2; t++) {
            const v4i v = {(int)pk[j][4 * t], (int)pk[j][4 * t + 1], (int)pk[j][4 * t + 2], (int)pk[j][4 * t + 3]};
            if (!EDGE || (row_l + i * 32 < rows_a && col_l + j * 32 + t * 16 < rows_b))
              __builtin_amdgcn_raw_buffer_store_b128(v, rC, voff + j * 64 + t * 32, i * 32 * N2, 0);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      const int col_l = wn * (TN * 32) + 4 * h;
      const int voff = row_l * N2 + col_l * 4;
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int gq = 0; gq < 4; gq++) {
            const v4f f = {acc[i][j][4 * gq], acc[i][j][4 * gq + 1], acc[i][j][4 * gq + 2], acc[i][j][4 * gq + 3]};
            if (!EDGE || (row_l + i * 32 < rows_a && col_l + j * 32 + gq * 8 < rows_b))
              __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, f), rC, voff + j * 128 + gq * 32, i * 32 * N2, 0);
          }
    }
  };

  // ---- all output tiles of this workgroup
  auto run = [&]<int GRP>() __attribute__((always_inline)) {
    for (;;) {
      k_loop.template operator()<GRP>();
      if constexpr (FUSED) fuse();
      {
        const auto g = fresh_args();
        const int rows_a = min(kBM, g->M - (tile_cur & 0xffff) * kBM), rows_b = min(kBN, g->N - (tile_cur >> 16) * kBN);
        if (rows_a == kBM && rows_b == kBN) epilogue.template operator()<false>(rows_a, rows_b);
        else epilogue.template operator()<true>(rows_a, rows_b);
      }
      if (tile_next < 0) break;
      p0 = (p0 + nk4) & 1;
      tile_cur = tile_next;
      bid_cur = bid_next;
      bid_next += gridDim.x;
      tile_next = tile_of(bid_next);
    }
  };

#ifdef MXFP6_PROBES
  auto clock_stamp = [&](int where) __attribute__((always_inline)) {
    const auto g = fresh_args();
    uint32_t* st = g->stamps;
    if (st && blockIdx.x == 0 && threadIdx.x == 0) {
      uint64_t t, r;
      asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t), "=s"(r)::"memory");
      st[2 * where] = (uint32_t)t, st[2 * where + 1] = (uint32_t)r;
    }
  };
#else
  auto clock_stamp = [](int) __attribute__((always_inline)) {};
#endif
  clock_stamp(0);
  // prologue: scales of the first four K-tiles, K-tiles 0 .. D-1 and, for group 1, the loads of tile D
  // that its compute cluster of "step -1" would have issued; tile 0 must have landed everywhere
  issue_scales.template operator()<true>(0);
  if (wm == 1) {
#pragma unroll
    for (int n = 0; n < S::NL1; n++) issue_one.template operator()<true, 1>(0, 0, n);
#pragma unroll
    for (int t = 1; t < D; t++)
#pragma unroll
      for (int n = 0; n < S::NL1; n++) issue_one.template operator()<false, 1>(t, t, n);
#pragma unroll
    for (int n = 0; n < kLoadsInCompute; n++) issue_one.template operator()<false, 1>(D, D, n);
    wait_vmcnt<(D - 1) * S::NL1 + kLoadsInCompute>();
  } else {
#pragma unroll
    for (int n = 0; n < S::NL; n++) issue_one.template operator()<true, 0>(0, 0, n);
#pragma unroll
    for (int t = 1; t < D; t++)
#pragma unroll
      for (int n = 0; n < S::NL; n++) issue_one.template operator()<false, 0>(t, t, n);
    wait_vmcnt<(D - 1) * S::NL>();
  }
  barrier();
  abl_started = true;
  if (wm == 0) {
    run.template operator()<0>();
    barrier();  // every wave executes the same number of barriers
  } else {
    barrier();  // phase offset of group 1
    run.template operator()<1>();
  }
  wait_vmcnt<0>();  // no direct load may still be on its way into LDS when the workgroup gives the memory back
  clock_stamp(1);
}

#ifndef MXFP6_TILED_FMT  // ---------------------------------------------------------------- the host-side object

bool gemm_tiled_supports(const GemmArgs& g) {
  // any M; N % 8 keeps every run of 8 bf16 outputs whole and aligned; K in whole K-tiles; 32-bit byte
  // offsets inside one tile's operand rows and inside one tile's rows of C
  return g.M > 0 && g.N > 0 && g.K > 0 && g.N % 8 == 0 && g.K % kBK == 0 && (long)256 * (g.K / 4 * 3) < (1L << 31) &&
         (long)256 * g.N * 4 < (1L << 31) && g.M <= 65535 * 128 && ((uintptr_t)g.C % 16) == 0 && operands_aligned16(g);
}

static int cu_count() {
  static int cus[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    cus[dev] = n;
  }
  return cus[dev];
}

// Workgroups to launch: one per output tile, or, when the tiles outnumber the compute units (one
// workgroup of this kernel fills a CU's LDS), one per CU, each walking through several tiles.  The
// scales of the next output tile are fetched with the last group of four K-tiles of the current one
// and must have two steps to land: K-tile counts of 4n+1 (and fewer than four K-tiles) keep one
// workgroup per tile.
int tiled_grid_size(const GemmArgs& g, int tiles, int per_cu) {
  const int cus = (cu_count() & ~7) * per_cu;  // whole multiples of the 8 XCDs keep the tile -> XCD mapping of the walk
  const int nkt = g.K / kBK;
  if (g_tiled_walk == 0 || nkt < 4 || nkt % 4 == 1 || cus < 8) return tiles;
  return tiles < cus ? tiles : cus;
}

// Sum of the K split's partial matrices, in share order, with the epilogue: 4 consecutive outputs per thread.
template <typename T>
__global__ __launch_bounds__(256) void ksplit_reduce_kernel(const float* __restrict__ part, int nsplit, T* __restrict__ C, int M, int N, const Epilogue ep) {
  const size_t mn = (size_t)M * N, i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i4 >= mn) return;
  v4f acc = *reinterpret_cast<const v4f*>(part + i4);
  for (int s = 1; s < nsplit; s++) {
    const v4f p = *reinterpret_cast<const v4f*>(part + s * mn + i4);
    acc += p;
  }
  const long m = (long)(i4 / N), n = (long)(i4 % N);
  if (epilogue_any(ep)) {
#pragma unroll
    for (int e = 0; e < 4; e++) acc[e] = epilogue_apply(ep, acc[e], m, n + e);
  }
  if constexpr (sizeof(T) == 2) {
    *reinterpret_cast<u32x2*>(C + i4) = u32x2{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3])};
  } else {
    *reinterpret_cast<v4f*>(C + i4) = acc;
  }
}

hipError_t launch_ksplit_reduce(const GemmArgs& g, hipStream_t s) {
  const size_t quads = (size_t)g.M * g.N / 4;
  const unsigned blocks = (unsigned)((quads + 255) / 256);
  if (g.f32out) ksplit_reduce_kernel<float><<<blocks, 256, 0, s>>>(g.ks_part, g.ksplit, (float*)g.C, g.M, g.N, g.ep);
  else ksplit_reduce_kernel<uint16_t><<<blocks, 256, 0, s>>>(g.ks_part, g.ksplit, (uint16_t*)g.C, g.M, g.N, g.ep);
  return hipGetLastError();
}

hipError_t launch_gemm_tiled(const GemmArgs& g, hipStream_t s) {
  if (g.fmt_a == 2 && g.fmt_b == 2) return launch_gemm_tiled_fmt22(g, s);
  if (g.fmt_a == 2 && g.fmt_b == 3) return launch_gemm_tiled_fmt23(g, s);
  if (g.fmt_a == 3 && g.fmt_b == 2) return launch_gemm_tiled_fmt32(g, s);
  if (g.fmt_a == 3 && g.fmt_b == 3) return launch_gemm_tiled_fmt33(g, s);
  return hipErrorInvalidValue;
}

#else  // ----------------------------------------------------------------------------------- one pair of operand formats

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  const bool ksplit = g.ksplit > 1 && g.ks_part;
  // the tile shape is the caller's (the dispatcher's choice, or a forced one); 256 x 256 unless told otherwise
  const int bm = g.tile_rows == 128 ? 128 : 256, bn = !ksplit && g.tile_cols == 128 && bm == 128 && !g.fmt_c ? 128 : 256;
  const int tm = (g.M + bm - 1) / bm, tn = (g.N + bn - 1) / bn;
  const TiledArgs ta = {g.A, g.B, g.As, g.Bs, g.C, g.M, g.N, g.K, tm, tn, g.layout_a, g.layout_b, g.ep, g.C_scale, g.fmt_c, g.raster_group_m > 0 ? g.raster_group_m : kGroupM, g.raster_no_xcd_remap == 1 ? 0 : g.raster_no_xcd_remap == 2 ? 2 : 1, ksplit ? g.ksplit : 1
#ifdef MXFP6_PROBES
                        , g.clock_stamps
#endif
  };
  if (ksplit) {
    if constexpr (sizeof(typename Out::type) != 1) {
      if ((bm != 128 && bm != 256) || g.K % (4 * kBK * g.ksplit) != 0 || g.K / kBK / g.ksplit < kMinShareTiles || (size_t)g.M * g.N % 4) return hipErrorInvalidValue;
      TiledArgs tp = ta;  // the shares write fp32 partial matrices into the workspace, without the epilogue
      tp.C = g.ks_part, tp.ep = Epilogue{};
      const int grid = tiled_grid_size(g, tm * tn * g.ksplit, 1);
      if (bm == 128) gemm_tiled_kernel<FA, FB, OutF32, 2, 2, false, 0, true><<<grid, NW * 64, 0, s>>>(tp);
      else gemm_tiled_kernel<FA, FB, OutF32, 4, 2, false, 0, true><<<grid, NW * 64, 0, s>>>(tp);
      const hipError_t e = hipGetLastError();
      return e != hipSuccess ? e : launch_ksplit_reduce(g, s);
    } else {
      return hipErrorInvalidValue;
    }
  }
  const int grid = tiled_grid_size(g, tm * tn, bn == 128 ? 2 : 1);  // 128 x 128: 80 KB of LDS, two workgroups per CU
  if constexpr (sizeof(typename Out::type) == 1) {  // fp6 output: one instantiation, with the fused step (a no-op when nothing is fused)
    if (bm == 128) gemm_tiled_kernel<FA, FB, Out, 2, 2, true><<<grid, NW * 64, 0, s>>>(ta);
    else gemm_tiled_kernel<FA, FB, Out, 4, 2, true><<<grid, NW * 64, 0, s>>>(ta);
  } else if (epilogue_any(g.ep)) {
    if (bn == 128) gemm_tiled_kernel<FA, FB, Out, 2, 1, true><<<grid, NW * 64, 0, s>>>(ta);
    else if (bm == 128) gemm_tiled_kernel<FA, FB, Out, 2, 2, true><<<grid, NW * 64, 0, s>>>(ta);
    else gemm_tiled_kernel<FA, FB, Out, 4, 2, true><<<grid, NW * 64, 0, s>>>(ta);
#ifdef MXFP6_PROBES
  } else if (g.ablation > 0 && g.ablation <= 8) {
    // measurement instantiations: e2m3 x e2m3, bf16 output, 256 x 256 tiles only
    if constexpr (FA == 2 && FB == 2 && sizeof(typename Out::type) == 2) {
      if (bm != 256 || bn != 256) return hipErrorInvalidValue;
      switch (g.ablation) {
        case 1: gemm_tiled_kernel<2, 2, Out, 4, 2, false, 1><<<grid, NW * 64, 0, s>>>(ta); break;
        case 2: gemm_tiled_kernel<2, 2, Out, 4, 2, false, 2><<<grid, NW * 64, 0, s>>>(ta); break;
        case 3: gemm_tiled_kernel<2, 2, Out, 4, 2, false, 3><<<grid, NW * 64, 0, s>>>(ta); break;
        case 4: gemm_tiled_kernel<2, 2, Out, 4, 2, false, 4><<<grid, NW * 64, 0, s>>>(ta); break;
        case 6: gemm_tiled_kernel<2, 2, Out, 4, 2, false, 6><<<grid, NW * 64, 0, s>>>(ta); break;
        case 8: gemm_tiled_kernel<2, 2, Out, 4, 2, false, 8><<<grid, NW * 64, 0, s>>>(ta); break;
        default: return hipErrorInvalidValue;  // 5 and 7 (no LDS reads and no MFMAs at once) are not built: the register allocator spills in them, which is all they would measure
      }
    } else {
      return hipErrorInvalidValue;
    }
#endif
  } else {
    if (bn == 128) gemm_tiled_kernel<FA, FB, Out, 2, 1, false><<<grid, NW * 64, 0, s>>>(ta);
    else if (bm == 128) gemm_tiled_kernel<FA, FB, Out, 2, 2, false><<<grid, NW * 64, 0, s>>>(ta);
    else gemm_tiled_kernel<FA, FB, Out, 4, 2, false><<<grid, NW * 64, 0, s>>>(ta);
  }
  return hipGetLastError();
}

#define MXFP6_PASTE2(a, b) a##b
#define MXFP6_PASTE(a, b) MXFP6_PASTE2(a, b)
hipError_t MXFP6_PASTE(launch_gemm_tiled_fmt, MXFP6_TILED_FMT)(const GemmArgs& g, hipStream_t s) {
  constexpr int FA = MXFP6_TILED_FMT / 10, FB = MXFP6_TILED_FMT % 10;
  static_assert((FA == 2 || FA == 3) && (FB == 2 || FB == 3), "MXFP6_TILED_FMT: 22, 23, 32 or 33");
  return g.fmt_c ? launch<FA, FB, OutFp6>(g, s) : g.f32out ? launch<FA, FB, OutF32>(g, s) : launch<FA, FB, OutBf16>(g, s);
}
#undef MXFP6_PASTE
#undef MXFP6_PASTE2

#endif  // MXFP6_TILED_FMT

}  // namespace mxfp6
