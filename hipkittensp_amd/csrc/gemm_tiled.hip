// LDS-tiled MXFP6 GEMM for gfx950: 256x256 output tile per workgroup, K-tile 128, 8 waves.
//
// Data path (no operand byte ever passes through a VGPR on its way to LDS):
//   global --buffer_load_dwordx4 ... lds--> LDS (3-stage ring) --ds_read_b128--> MFMA source VGPRs
//   v_mfma_scale_f32_32x32x64_f8f6f4 (fp32 accumulate, E8M0 block scales applied by the instruction)
//   accumulators --v_cvt_pk_bf16_f32--> LDS --> whole rows to global
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
// load per 64 rows per four K-tiles; a lane reads the 2 bytes it needs with ds_read_u16 and the MFMA's
// op_sel picks byte 0 / byte 1.
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
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

constexpr int kBM = 256, kBN = 256, kBK = 128;
constexpr int kOpStage = 256 * 96;  // bytes of one operand tile
constexpr int kScStage = 256 * 16;  // bytes of one operand's scales for four K-tiles
constexpr int kGroupM = 4;          // tile rows per raster group
constexpr int kStages = 3;          // operand ring depth
constexpr int kStage = 2 * kOpStage, kScaleBase = kStages * kStage, kScaleBuf = 2 * kScStage;
constexpr int kLdsBytes = kScaleBase + 2 * kScaleBuf;
constexpr int WM = 2, WN = 4, NW = WM * WN;  // waves: 2 x 4, wave tile 128 x 64
constexpr int TM = 8 / WM, TN = 8 / WN;      // 32x32 MFMA tiles per wave in M and N
constexpr int OPS = 24 / NW;                 // operand direct loads per wave per operand per K-tile
constexpr int SCL = 1;                       // scale direct loads per wave per slot that carries scales
constexpr int kLoadsInCompute = 4;           // of the 2*OPS operand loads per wave and K-tile: issued between MFMAs
static_assert(kLoadsInCompute >= 0 && kLoadsInCompute <= 2 * OPS && 2 * kLoadsInCompute <= 2 * TM * TN, "load slots");
static_assert(kLdsBytes <= 163840, "LDS budget");

// One direct-to-LDS load: every lane fetches 16 bytes at rsrc.base + voff + soff and the hardware
// writes them at LDS address lds_base + 16 * lane.  Issued from inline assembly so that the VMEM
// counter is managed by hand: the ring keeps two K-tiles in flight across barriers, which the
// compiler's automatic waits would serialise.  M0 is used by nothing else in this kernel.
__device__ __forceinline__ void dma16(const __amdgpu_buffer_rsrc_t& rsrc, uint32_t lds_base, int voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void barrier() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

template <int FA, int FB, typename Out>
__global__ __launch_bounds__(NW * 64) void gemm_tiled_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                             const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bs,
                                                             typename Out::type* __restrict__ C, int M, int N, int K,
                                                             int tiles_m, int tiles_n, int layout_a, int layout_b) {
  // LDS map: [stage 0..2][A tile | B tile] then [scale buffer 0..1][A scales | B scales]
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kLdsBytes];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem;

  // ---- workgroup -> output tile: undo the round-robin XCD placement, then a grouped raster.
  // Hardware places workgroup b on XCD b % 8; remapping gives each XCD a contiguous run of logical
  // tiles so that the 32 tiles an XCD works on at once share operand rows in its L2
  // (the idea of chiplet_transform_chunked, include/common/util.cuh:78-101, as an exact bijection).
  const int nb = tiles_m * tiles_n;
  int L;
  {
    const int bid = blockIdx.x, xcd = bid & 7, idx = bid >> 3;
    const int per = nb >> 3, rem = nb & 7;
    L = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
  }
  int pm, pn;
  {
    const int width = kGroupM * tiles_n, group = L / width, first = group * kGroupM;
    const int gsz = min(tiles_m - first, kGroupM), in = L - group * width;
    pm = first + in % gsz;
    pn = in / gsz;
  }

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int h = lane >> 5, r32 = lane & 31;

  const int rowbytes = K / 4 * 3, sbytes = K / 32, nkt = K / kBK;
  // edge tiles: rows past M (or N) lie beyond the end of the buffer resource and read as zeros
  const int rows_a = min(kBM, M - pm * kBM), rows_b = min(kBN, N - pn * kBN);
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A + (size_t)pm * kBM * rowbytes, (uint32_t)rows_a * rowbytes);
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(B + (size_t)pn * kBN * rowbytes, (uint32_t)rows_b * rowbytes);
  // tile-major scales: the 16 bytes a row has for four K-tiles, 32 rows adjacent (512-byte chunks, nk4 per row-tile)
  const int nk4 = (nkt + 3) / 4;
  const __amdgpu_buffer_rsrc_t rSA = layout_a ? make_rsrc(As + (size_t)pm * (kBM / 32) * nk4 * 512, (uint32_t)((rows_a + 31) / 32) * nk4 * 512)
                                              : make_rsrc(As + (size_t)pm * kBM * sbytes, (uint32_t)rows_a * sbytes);
  const __amdgpu_buffer_rsrc_t rSB = layout_b ? make_rsrc(Bs + (size_t)pn * (kBN / 32) * nk4 * 512, (uint32_t)((rows_b + 31) / 32) * nk4 * 512)
                                              : make_rsrc(Bs + (size_t)pn * kBN * sbytes, (uint32_t)rows_b * sbytes);

  // per-lane global byte offsets of the OPS direct loads.  Load q = wave*OPS + i fills LDS bytes
  // [q*1024, q*1024 + 1024) of the operand tile.  Row-major operand: slot o holds piece
  // (o%6) ^ ((row>>3)&1) of row o/6, K-tile t starts at byte 96 t of a row.  Tile-major operand:
  // the 3072-byte tile of 32 rows is stored in exactly this order, so the load is one contiguous
  // KiB, row-tiles are (K/128)*3072 bytes apart and K-tile t starts at byte 3072 t.
  int voff_a[OPS], voff_b[OPS];
#pragma unroll
  for (int i = 0; i < OPS; i++) {
    const int q = wave * OPS + i, o = q * 64 + lane;  // linear 16-byte slot inside the LDS image
    const int r = o / 6, c = (o - r * 6) ^ ((r >> 3) & 1);
    const int vrow = r * rowbytes + c * 16;
    const int vtile = (q / 3) * (nkt * 3072) + (q % 3) * 1024 + lane * 16;
    voff_a[i] = layout_a ? vtile : vrow;
    voff_b[i] = layout_b ? vtile : vrow;
  }
  const int kstep_a = layout_a ? 3072 : 96, kstep_b = layout_b ? 3072 : 96;
  // scales: a lane fetches the 16 scale bytes (four K-tiles) of one row; waves 0-3 load A's, 4-7 B's
  const int srow = (wave & 3) * 64 + lane, slay = wave < 4 ? layout_a : layout_b;
  const int voff_s = slay ? (srow >> 5) * nk4 * 512 + (srow & 31) * 16 : srow * sbytes;
  const int sstep = slay ? 512 : 16;  // bytes between consecutive groups of four K-tiles

  // per-lane LDS read offsets (bytes from the start of a stage): the lane's three pieces 3h..3h+2
  const int sw = (r32 >> 3) & 1;
  int a_rd[3], b_rd[3];
#pragma unroll
  for (int c = 0; c < 3; c++) {
    a_rd[c] = (wm * (TM * 32) + r32) * 96 + ((3 * h + c) ^ sw) * 16;
    b_rd[c] = kOpStage + (wn * (TN * 32) + r32) * 96 + ((3 * h + c) ^ sw) * 16;
  }
  const int sa_rd = kScaleBase + (wm * (TM * 32) + r32) * 16 + 2 * h;
  const int sb_rd = kScaleBase + kScStage + (wn * (TN * 32) + r32) * 16 + 2 * h;

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

  // ---- loads.  A wave's batch for K-tile t is its 2*OPS operand loads (n = 0..OPS-1: A, then B) and,
  // when t % 4 == 2, the scale load for the four K-tiles starting at t + 2 (at the end of the batch, so
  // that a wait that leaves a whole batch in flight also covers the scales of the batch before).
  auto issue_scales = [&](int grp) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + kScaleBase + (grp & 1) * kScaleBuf + (wave & 3) * 1024;
    const int soff = grp * sstep;
    if (wave < 4) dma16(rSA, dst, voff_s, soff); else dma16(rSB, dst + kScStage, voff_s, soff);
  };
  auto issue_one = [&](int t, int slot, int n) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + slot * kStage + wave * (OPS * 1024);
    if (n < OPS) dma16(rA, dst + n * 1024, voff_a[n], t * kstep_a);
    else dma16(rB, dst + kOpStage + (n - OPS) * 1024, voff_b[n - OPS], t * kstep_b);
  };
  auto issue_ops = [&](int t, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < 2 * OPS; n++) issue_one(t, slot, n);
  };

  // ---- one K-tile: LDS -> registers (memory cluster) and the MFMAs (compute cluster)
  // a lane's 48 bytes of one 32-row tile live in 12 consecutive VGPRs: dwords 0-5 are the operand of the
  // first MFMA, 6-11 of the second
  v12i fa[TM], fb[TN];
  int sca[TM], scb[TN];
  auto read_tile = [&](int stage, int sc_off) __attribute__((always_inline)) {
    const uint8_t* st = smem + stage * kStage;
    const uint8_t* sc = smem + sc_off;
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const v4i p = *reinterpret_cast<const v4i*>(st + b_rd[c] + j * 3072);
#pragma unroll
        for (int e = 0; e < 4; e++) fb[j][4 * c + e] = p[e];
      }
      scb[j] = *reinterpret_cast<const uint16_t*>(sc + sb_rd + j * 512);
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const v4i p = *reinterpret_cast<const v4i*>(st + a_rd[c] + i * 3072);
#pragma unroll
        for (int e = 0; e < 4; e++) fa[i][4 * c + e] = p[e];
      }
      sca[i] = *reinterpret_cast<const uint16_t*>(sc + sa_rd + i * 512);
    }
  };
  // first K-block of every lane for all tiles, then the second: two MFMAs into the same accumulator
  // are TM*TN instructions apart.  First source = B rows (index n), second = A rows (index m): a
  // lane ends up owning 4 consecutive n of one m.  between(i) runs after the i-th MFMA.
  auto mma_tile = [&](auto&& between) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const v8i a0 = __builtin_shufflevector(fa[i], fa[i], 0, 1, 2, 3, 4, 5, -1, -1);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const v8i b0 = __builtin_shufflevector(fb[j], fb[j], 0, 1, 2, 3, 4, 5, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc[i][j], scb[j], sca[i]);
        between(i * TN + j);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const v8i a1 = __builtin_shufflevector(fa[i], fa[i], 6, 7, 8, 9, 10, 11, -1, -1);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const v8i b1 = __builtin_shufflevector(fb[j], fb[j], 6, 7, 8, 9, 10, 11, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc[i][j], scb[j], sca[i]);
        between(TM * TN + i * TN + j);
      }
    }
  };

  // ---- the K loop.  Barrier n is common to all waves; between barriers 2k and 2k+1 group 0 (waves
  // 0-3) is in its memory cluster for tile k and between 2k+1 and 2k+2 in its compute cluster; group 1
  // (waves 4-7) does the same one barrier later.  A ring slot is refilled only after the barrier by
  // which both groups have finished reading it, and each wave waits for its own share of tile k+1
  // before the barrier that precedes the first read of that tile.
  // Loads of step k.  Memory cluster, after the LDS reads, both groups: loads kLoadsInCompute.. of tile
  // k+2 (slot of tile k-1, free since barrier 2k) and the scales.  Compute cluster: loads
  // 0..kLoadsInCompute-1, for group 0 of the same tile k+2, for group 1 of tile k+3, whose slot is the
  // one of tile k: group 1's compute cluster starts at barrier 2k+2, by which both groups have read
  // tile k.  In program order every tile's batch is contiguous for both groups, so one wait count
  // serves both: everything older than the newest batch has landed.
  // The body is instantiated per group (GRP) and per k mod 4 (KM), so the steady state carries no
  // branch: STEADY means tiles k+2, k+3 and (for the scales) k+4 exist.
  int stage = 0, stage2 = 2;  // ring slots of tile k and tile k+2
  auto step = [&]<int GRP, int KM, bool STEADY>(int kt) __attribute__((always_inline)) {
    constexpr int AHEAD = GRP == 0 ? 2 : 3;
    const bool has2 = STEADY || kt + 2 < nkt;             // tile kt+2 exists
    const bool hasx = STEADY || kt + AHEAD < nkt;         // the tile the compute-cluster loads belong to exists
    const bool has_sc = STEADY || kt + 4 < nkt;           // the scales this step's batch would carry exist
    const int slotx = GRP == 0 ? stage2 : stage;
    read_tile(stage, ((kt >> 2) & 1) * kScaleBuf + KM * 4);
    __builtin_amdgcn_sched_barrier(0);
    if (has2) {
#pragma unroll
      for (int n = kLoadsInCompute; n < 2 * OPS; n++) issue_one(kt + 2, stage2, n);
      if (KM == 0 && has_sc) issue_scales((kt + 4) >> 2);
    }
    wait_lds_reads();  // this tile's LDS reads are done before anyone may refill its slot
    // the middle 16-byte piece straddles the two operands; naming each fragment as one 384-bit value here
    // makes the register allocator keep it in one tuple, and the MFMAs read sub-tuples of it instead of
    // copies (24 v_mov per K-tile otherwise)
#pragma unroll
    for (int i = 0; i < TM; i++) asm volatile("" : "+v"(fa[i]));
#pragma unroll
    for (int j = 0; j < TN; j++) asm volatile("" : "+v"(fb[j]));
    auto wait_next = [&]() __attribute__((always_inline)) {  // own share of tile kt+1 has landed; tile kt+2's batch may be in flight
      if (has2) {
        if (KM == 0 && has_sc) wait_vmcnt<2 * OPS + SCL>(); else wait_vmcnt<2 * OPS>();
      } else {
        wait_vmcnt<0>();
      }
    };
    if (GRP == 1) wait_next();
    barrier();
    __builtin_amdgcn_s_setprio(1);
    mma_tile([&](int i) __attribute__((always_inline)) {
      if (hasx && (i & 1) && i / 2 < kLoadsInCompute) {
        __builtin_amdgcn_sched_barrier(0);
        issue_one(kt + AHEAD, slotx, i / 2);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    __builtin_amdgcn_s_setprio(0);
    if (GRP == 0) wait_next();
    barrier();
    stage = stage == kStages - 1 ? 0 : stage + 1;
    stage2 = stage2 == kStages - 1 ? 0 : stage2 + 1;
  };
  auto k_loop = [&]<int GRP>() __attribute__((always_inline)) {
    int kt = 0;
    for (; kt + 8 <= nkt; kt += 4) {  // four tiles per trip, all of them with tiles kt+2 .. kt+7 in range
      step.template operator()<GRP, 0, true>(kt);
      step.template operator()<GRP, 1, true>(kt + 1);
      step.template operator()<GRP, 2, true>(kt + 2);
      step.template operator()<GRP, 3, true>(kt + 3);
    }
    for (; kt < nkt; kt += 4) {  // last (up to seven) tiles: same body with the range checks
      step.template operator()<GRP, 0, false>(kt);
      if (kt + 1 < nkt) step.template operator()<GRP, 1, false>(kt + 1);
      if (kt + 2 < nkt) step.template operator()<GRP, 2, false>(kt + 2);
      if (kt + 3 < nkt) step.template operator()<GRP, 3, false>(kt + 3);
    }
  };

  // prologue: scales of the first four K-tiles, K-tiles 0 and 1 and, for group 1, the loads of tile 2
  // that its compute cluster of "step -1" would have issued; tile 0 must have landed everywhere
  issue_scales(0);
  issue_ops(0, 0);
  if (nkt > 1) issue_ops(1, 1);
  if (wm == 1 && nkt > 2 && kLoadsInCompute > 0) {
#pragma unroll
    for (int n = 0; n < kLoadsInCompute; n++) issue_one(2, 2, n);
    wait_vmcnt<2 * OPS + kLoadsInCompute>();
  } else if (nkt > 1) {
    wait_vmcnt<2 * OPS>();
  } else {
    wait_vmcnt<0>();
  }
  barrier();
  if (wm == 0) {
    k_loop.template operator()<0>();
    barrier();  // every wave executes the same number of barriers
  } else {
    barrier();  // phase offset of group 1
    k_loop.template operator()<1>();
  }

  // ---- epilogue.  A lane owns C[m][n .. n+3] for four values of n per 32x32 tile, i.e. 8 bytes of
  // bf16 per store: written straight to global memory those are partial-line writes (measured 1.4x
  // the output in HBM write traffic and a visible tail after every tile).  The bf16 tile (128 KB)
  // is therefore staged through LDS, which is free once the K loop is over, and written out in
  // whole rows: one wave store = two rows x 512 contiguous bytes.
  if constexpr (sizeof(typename Out::type) == 2) {
    constexpr int kRowPitch = 512 + 16;  // bytes; the pad spreads the 32 rows of a store over the banks
    static_assert(256 * kRowPitch <= kLdsBytes, "C tile fits the ring");
    __syncthreads();  // every wave is done reading the ring
    uint8_t* cs = smem + (wm * (TM * 32) + r32) * kRowPitch + (wn * (TN * 32) + 4 * h) * 2;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const u32x2 v = {pack_bf16x2(acc[i][j][4 * g], acc[i][j][4 * g + 1]), pack_bf16x2(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3])};
          *reinterpret_cast<u32x2*>(cs + i * 32 * kRowPitch + (j * 32 + 8 * g) * 2) = v;
        }
    __syncthreads();
    const int chunk = tid & 31, row0 = tid >> 5;  // 32 lanes cover one 512-byte row
    uint8_t* cg = reinterpret_cast<uint8_t*>(C) + ((size_t)pm * kBM + row0) * (size_t)N * 2 + (size_t)pn * kBN * 2 + chunk * 16;
    constexpr int kRowsPerPass = NW * 2;
    const bool col_ok = chunk * 8 < rows_b;  // N % 8 == 0: a 16-byte piece is inside or outside as a whole
#pragma unroll 4
    for (int r = 0; r < 256; r += kRowsPerPass) {
      const v4i v = *reinterpret_cast<const v4i*>(smem + (row0 + r) * kRowPitch + chunk * 16);
      if (col_ok && row0 + r < rows_a) *reinterpret_cast<v4i*>(cg + (size_t)r * N * 2) = v;
    }
  } else {
    typename Out::type* cbase = C + ((size_t)pm * kBM + wm * (TM * 32) + r32) * (size_t)N + (size_t)pn * kBN + wn * (TN * 32) + 4 * h;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++)
          if (wm * (TM * 32) + i * 32 + r32 < rows_a && wn * (TN * 32) + j * 32 + 8 * g + 4 * h < rows_b)
            store4(cbase + (size_t)i * 32 * N + j * 32 + 8 * g, acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                   acc[i][j][4 * g + 3]);
  }
}

bool gemm_tiled_supports(const GemmArgs& g) {
  // any M; N % 8 keeps every 16-byte output piece whole and aligned; K in whole K-tiles
  return g.M > 0 && g.N > 0 && g.K > 0 && g.N % 8 == 0 && g.K % kBK == 0 && (long)kBM * (g.K / 4 * 3) < (1L << 31) &&
         ((uintptr_t)g.C % 16) == 0;
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  const int tm = (g.M + kBM - 1) / kBM, tn = (g.N + kBN - 1) / kBN;
  gemm_tiled_kernel<FA, FB, Out><<<tm * tn, NW * 64, 0, s>>>(g.A, g.B, g.As, g.Bs, (typename Out::type*)g.C, g.M, g.N, g.K, tm, tn,
                                                            g.layout_a, g.layout_b);
  return hipGetLastError();
}

hipError_t launch_gemm_tiled(const GemmArgs& g, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (g.fmt_a == FA && g.fmt_b == FB) return g.f32out ? launch<FA, FB, OutF32>(g, s) : launch<FA, FB, OutBf16>(g, s);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipErrorInvalidValue;
}

}  // namespace mxfp6
