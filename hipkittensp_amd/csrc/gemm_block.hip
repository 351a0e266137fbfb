// MXFP6 GEMM for a few hundred to a few thousand rows of A: output tiles of 128 x 128, four waves in step.
//
// The 8-wave ping-pong kernel (gemm_tiled.hip) alternates two wave groups between a memory cluster and a compute
// cluster, which pays when a compute cluster is as long as a memory cluster: 16 MFMAs per wave and K-tile at 256 x 256.
// With the small tiles that fill the machine at a few hundred rows of A a compute cluster is 4 MFMAs, and a K-tile costs
// the two memory clusters one after the other: the operand fragments' way from LDS into registers, twice, plus two
// barriers.  Here nothing alternates.  Every wave owns a 64 x 64 corner of the tile (2 x 2 MFMA tiles, both K-steps of a
// K-tile: 8 MFMAs per K-tile) and keeps two sets of fragment registers: while the MFMAs of K-tile k run on one set, the
// LDS reads of K-tile k+1 fill the other and the direct loads of K-tile k+3 go out; one barrier per K-tile.  48 KB of LDS
// reads per K-tile and workgroup (the 8-wave kernel's 128 x 128 shape: 72 KB).  80 KB of LDS: two workgroups per CU,
// one's waits are the other's work.
//
// Same operand formats, LDS image, lane mapping and raster as the tiled kernel (common.hpp, gemm_tiled.hip): row-major
// or tile-major operands and scales, any M and N (edge tiles: rows past M or N lie beyond the end of their buffer
// resource and read as zeros, stores are predicated), K % 128 == 0, bf16 or fp32 output, fused scales / bias / activation
// (separate instantiations).
//   ring: three slots of 24 KB (A's 128 rows x 96 bytes, then B's); K-tile k lives in slot k % 3
//   scales: the 16 bytes a row has for four K-tiles, two buffers of (128 + 128) rows x 16 bytes, group g in buffer g % 2
//   step k: loads of K-tile k+3 into the slot K-tile k has left (its fragments are in registers since step k-1), LDS
//           reads of K-tile k+1, MFMAs of K-tile k, wait for the LDS reads and for every load older than this step's,
//           barrier.  A load has two steps to land.
#include "kernels.hpp"
#include "loader.hpp"

namespace mxfp6 {
namespace {

constexpr int kBM = 128, kBK = 128;
constexpr int kATile = kBM * 96;  // bytes of A's tile in a ring slot
constexpr int kScA = kBM * 16;    // bytes of A's scales for four K-tiles
constexpr int kGroupM = 8;        // tile rows per raster group


struct BlockArgs {
  const uint8_t *A, *B, *As, *Bs;
  void* C;
  int M, N, K, tiles_m, tiles_n, layout_a, layout_b, group_m, xcd_remap;
  int nsplit;  // workgroups that share an output tile, each over the same number of whole groups of four K-tiles (the last one over what is left); 1 = no split
  Epilogue ep;  // FUSED instantiations: scales / bias / activation on the accumulators before the output rounding
};

// STAGES: ring slots, 3 (80 KB of LDS, two workgroups per CU) to 6 (152 KB, one).  Loads run STAGES K-tiles ahead of the
// MFMAs and have STAGES - 1 steps to land; from five slots on the scales are fetched two groups ahead instead of one, so
// that they are older than every load a step's wait leaves in flight.
// WN: waves side by side along N, 2 (tile of 128 x 128, four waves) or 4 (128 x 256, eight waves: waves 0-3 load A's tile
// and half of B's, six loads per K-tile, waves 4-7 the other half of B's, three loads).
// FUSED: the epilogue applies args.ep (a separate instantiation, so that unfused calls carry none of it).
template <int FA, int FB, typename Out, int STAGES, int WN, bool FUSED>
__global__ __launch_bounds__(2 * WN * 64, STAGES <= 3 ? 2 : WN / 2) void gemm_block_kernel(const BlockArgs args) {
  typedef typename Out::type OutT;
  static_assert(STAGES >= 3 && STAGES <= 6 && (WN == 2 || WN == 4), "ring depth, tile width");
  constexpr int NW = 2 * WN, kBN = WN * 64, kSlot = kATile + kBN * 96, kScBuf = kScA + kBN * 16;
  constexpr int kStages = STAGES, E = STAGES > 4 ? 1 : 0;  // E: extra groups of four K-tiles the scale loads run ahead
  constexpr int kScBase = kStages * kSlot, kLdsBytes = kScBase + 2 * kScBuf;
  static_assert(kLdsBytes <= (STAGES <= 3 && WN == 2 ? 81920 : 163840), "LDS budget");
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kLdsBytes];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem;
  const int K = args.K, layout_a = args.layout_a, layout_b = args.layout_b;
  const int rowbytes = K / 4 * 3, sbytes = K / 32, nkt_all = K / kBK, nk4_all = (nkt_all + 3) / 4;  // tile-major scales: one 512-byte chunk per 32 rows and group of four K-tiles, the last one padded
  // K split: workgroup b takes share l / tiles of tile l % tiles, l = ksplit_order(b) -- the same number of whole groups
  // of four K-tiles for every share, the last one what is left of K (at least one K-tile: the launcher sees to that) --
  // and leaves its fp32 sums in matrix `share` of args.C, then a workspace of nsplit matrices [M, N]
  // (ksplit_reduce_kernel adds them up)
  const int ntiles = args.tiles_m * args.tiles_n;
  const bool by_share = args.nsplit > 1 && ksplit_by_share(ntiles * args.nsplit, args.xcd_remap);  // the XCDs are dealt by ksplit_order, not by tile_order
  const int order = args.nsplit > 1 ? ksplit_order(blockIdx.x, ntiles * args.nsplit, args.xcd_remap) : blockIdx.x, share = order / ntiles;
  const int share_groups = (nk4_all + args.nsplit - 1) / args.nsplit, kt0 = share * share_groups * 4;
  const int nkt = min(nkt_all - kt0, share_groups * 4), nk4 = (nkt + 3) / 4;

  const int tile = tile_order(order - share * ntiles, args.tiles_m, args.tiles_n, args.group_m, by_share ? 0 : args.xcd_remap);
  if (tile < 0) return;  // never: the grid is the tile count times the shares
  const int pm = tile & 0xffff, pn = tile >> 16;
  const int rows_a = min(kBM, args.M - pm * kBM), rows_b = min(kBN, args.N - pn * kBN);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const bool loads_a = wave < 4;  // this wave loads row-tile `wave` of A's tile (every wave loads row-tile `wave` of B's)
  const int h = lane >> 5, r32 = lane & 31;

  // operand rows of this tile; rZ: a resource of length zero, loads through it fetch nothing (K-tiles past the end)
  // (a share's resources start at its first K-tile, 96 or 3072 bytes times kt0 into a row or row-tile, and end that much
  // earlier, so that rows past the tile's last still lie beyond the end)
  const uint32_t oa = (uint32_t)kt0 * (layout_a ? 3072 : 96), ob = (uint32_t)kt0 * (layout_b ? 3072 : 96);
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(args.A + (size_t)pm * kBM * rowbytes + oa, (uint32_t)rows_a * rowbytes - oa);
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(args.B + (size_t)pn * kBN * rowbytes + ob, (uint32_t)rows_b * rowbytes - ob);
  const __amdgpu_buffer_rsrc_t rZ = make_rsrc(args.A, 0);
  // scales: the first half of the waves fetch A's (rows 0-63, 64-127 of the tile; with eight waves, waves 2, 3 fetch what
  // waves 0, 1 fetch, into the same place, so that every wave issues one scale load per group), the second half B's, 64
  // rows each; a lane fetches the 16 bytes one row has for four K-tiles
  const bool sc_a = wave < NW / 2;
  const int slay = sc_a ? layout_a : layout_b, srows = sc_a ? rows_a : rows_b, stile = sc_a ? pm : pn;
  const uint8_t* sp = sc_a ? args.As : args.Bs;
  const int sheight = sc_a ? kBM : kBN;  // rows per tile of the operand whose scales these are
  const uint32_t os = (uint32_t)(kt0 >> 2) * (slay ? 512 : 16);  // the share's first group of four K-tiles
  const __amdgpu_buffer_rsrc_t rS = slay ? make_rsrc(sp + (size_t)stile * (sheight / 32) * nk4_all * 512 + os, (uint32_t)((srows + 31) / 32) * nk4_all * 512 - os)
                                         : make_rsrc(sp + (size_t)stile * sheight * sbytes + os, (uint32_t)srows * sbytes - os);
  const int spart = sc_a ? wave & 1 : wave - NW / 2;  // which 64 rows
  const int srow = spart * 64 + lane;
  const int voff_s = slay ? (srow >> 5) * nk4_all * 512 + (srow & 31) * 16 : srow * sbytes;
  const int sstep = slay ? 512 : 16;
  const uint32_t sdst = lds0 + kScBase + (sc_a ? 0 : kScA) + spart * 1024;

  // per-lane global byte offsets of the direct loads: load q = 3 wave + i fills LDS bytes [q * 1024, + 1024) of an
  // operand's tile.  Row-major: 16-byte slot o holds piece (o % 6) ^ ((row >> 3) & 1) of row o / 6.  Tile-major: the
  // 3072-byte tile of 32 rows is stored in this order; wave w loads row-tile w.
  int voff_a[3], voff_b[3];
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int q = wave * 3 + i, o = q * 64 + lane;
    const int r = o / 6, c = (o - r * 6) ^ ((r >> 3) & 1);
    const int vrow = r * rowbytes + c * 16, vtile = wave * (nkt_all * 3072) + i * 1024 + lane * 16;
    voff_a[i] = layout_a ? vtile : vrow;
    voff_b[i] = layout_b ? vtile : vrow;
  }
  const int kstep_a = layout_a ? 3072 : 96, kstep_b = layout_b ? 3072 : 96;

  // per-lane LDS read offsets inside a slot: the lane's three 16-byte pieces 3h .. 3h + 2 of its row
  const int sw = (r32 >> 3) & 1;
  int a_rd[3], b_rd[3];
#pragma unroll
  for (int c = 0; c < 3; c++) {
    a_rd[c] = (wm * 64 + r32) * 96 + ((3 * h + c) ^ sw) * 16;
    b_rd[c] = kATile + (wn * 64 + r32) * 96 + ((3 * h + c) ^ sw) * 16;
  }
  const int sa_rd = kScBase + (wm * 64 + r32) * 16, sb_rd = kScBase + kScA + (wn * 64 + r32) * 16;
  const int sc_shift = 16 * h;  // a lane's two scale bytes of a K-tile: bytes 2h, 2h + 1 of the K-tile's four

  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;
  v12i fa[2][2], fb[2][2];  // [set][tile]: a lane's 48 bytes of a 32-row tile, dwords 0-5 the first MFMA's operand, 6-11 the second's
  int sca[2][4], scb[2][4];  // [tile][K-tile of the group]: scale bytes in bytes 0, 1
  v4i raw_a[2], raw_b[2];

  // load n of this wave's for K-tile t: 0-2 the three of row-tile `wave` of A's tile (LA: this wave loads A at all), 3-5 of B's
  auto load_one = [&]<bool LA>(int t, int slot, int n) __attribute__((always_inline)) {
    const bool in = t < nkt;
    const uint32_t dst = lds0 + slot * kSlot + wave * 3072;
    if (n < 3) {
      if constexpr (LA) dma16(in ? rA : rZ, dst + n * 1024, voff_a[n], t * kstep_a);
    } else {
      dma16(in ? rB : rZ, dst + kATile + (n - 3) * 1024, voff_b[n - 3], t * kstep_b);
    }
  };
  auto load_tile = [&]<bool LA>(int t, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < 6; n++) load_one.template operator()<LA>(t, slot, n);
  };
  // (the group's offset goes into the per-lane offset, which the hardware checks against the end of the resource: with
  // K % 512 != 0 the last group of a row-major row is shorter than 16 bytes, and the last row's must not read past the tensor)
  auto load_scales = [&](int grp) __attribute__((always_inline)) {
    const __amdgpu_buffer_rsrc_t rs = grp < nk4 ? rS : rZ;
    dma16(rs, sdst + (grp & 1) * kScBuf, voff_s + grp * sstep, 0);
  };
  auto read_tile = [&]<int SET>(int slot) __attribute__((always_inline)) {
    const uint8_t* st = smem + slot * kSlot;
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const v4i p = *reinterpret_cast<const v4i*>(st + b_rd[c] + j * 3072);
#pragma unroll
        for (int e = 0; e < 4; e++) fb[SET][j][4 * c + e] = p[e];
      }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const v4i p = *reinterpret_cast<const v4i*>(st + a_rd[c] + i * 3072);
#pragma unroll
        for (int e = 0; e < 4; e++) fa[SET][i][4 * c + e] = p[e];
      }
  };
  auto read_scales = [&](int grp) __attribute__((always_inline)) {
    const uint8_t* sc = smem + (grp & 1) * kScBuf;
#pragma unroll
    for (int i = 0; i < 2; i++) raw_a[i] = *reinterpret_cast<const v4i*>(sc + sa_rd + i * 512);
#pragma unroll
    for (int j = 0; j < 2; j++) raw_b[j] = *reinterpret_cast<const v4i*>(sc + sb_rd + j * 512);
  };
  auto take_scales = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int km = 0; km < 4; km++) sca[i][km] = (int)((uint32_t)raw_a[i][km] >> sc_shift), scb[i][km] = (int)((uint32_t)raw_b[i][km] >> sc_shift);
  };
  // first source = B rows (index n), second = A rows (index m): a lane ends up owning 4 consecutive n of row m = lane % 32,
  // four times per 32 x 32 tile
  // between(q) runs after the q-th of the eight MFMAs
  auto mma_tile = [&]<int SET, int KM>(auto&& between) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const v8i a0 = __builtin_shufflevector(fa[SET][i], fa[SET][i], 0, 1, 2, 3, 4, 5, -1, -1);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const v8i b0 = __builtin_shufflevector(fb[SET][j], fb[SET][j], 0, 1, 2, 3, 4, 5, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc[i][j], scb[j][KM], sca[i][KM]);
        between(i * 2 + j);
      }
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const v8i a1 = __builtin_shufflevector(fa[SET][i], fa[SET][i], 6, 7, 8, 9, 10, 11, -1, -1);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const v8i b1 = __builtin_shufflevector(fb[SET][j], fb[SET][j], 6, 7, 8, 9, 10, 11, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc[i][j], scb[j][KM], sca[i][KM]);
        between(4 + i * 2 + j);
      }
    }
  };

  // slot[i]: ring slot of K-tile k + i
  int slot[kStages];
#pragma unroll
  for (int i = 0; i < kStages; i++) slot[i] = i;
  // LA: this wave loads A's tile too (six loads per K-tile, else three); instantiated per wave class, so that no branch
  // sits between the MFMAs (a branch there makes the compiler keep a second copy of the accumulators)
  auto step = [&]<int KM, bool LA>(int k) __attribute__((always_inline)) {
    constexpr int CUR = KM & 1, NXT = CUR ^ 1;
    // LDS reads of K-tile k + 1 first, then the MFMAs of K-tile k with the direct loads of K-tile k + STAGES (into K-tile
    // k's slot) between them, one after each of the first six, and after the seventh the scales of a later group of four
    // (with a group's first K-tile): the loads wait for the address unit behind an MFMA instead of in front of the LDS reads
    read_tile.template operator()<NXT>(slot[1]);
    if (KM == 3) read_scales((k >> 2) + 1);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(1);
    mma_tile.template operator()<CUR, KM>([&](int q) __attribute__((always_inline)) {
      __builtin_amdgcn_sched_barrier(0);
      if (q < 6) load_one.template operator()<LA>(k + kStages, slot[0], q);
      if (q == 6 && KM == 0) load_scales((k >> 2) + 1 + E);
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    wait_lds_reads();
#pragma unroll
    for (int i = 0; i < 2; i++) asm volatile("" : "+v"(fa[NXT][i]));
#pragma unroll
    for (int j = 0; j < 2; j++) asm volatile("" : "+v"(fb[NXT][j]));
    if (KM == 3) take_scales();
    // K-tile k + 2 has landed: everything older than the loads of the last STAGES - 2 steps (six each, and a scale load
    // in steps with KM == 0)
    constexpr int kScalesInFlight = (KM % 4 == 0) + (STAGES >= 4 && (KM + 3) % 4 == 0) + (STAGES >= 5 && (KM + 2) % 4 == 0) + (STAGES >= 6 && (KM + 1) % 4 == 0);
    wait_vmcnt<(LA ? 6 : 3) * (STAGES - 2) + kScalesInFlight>();
    barrier();
    const int t = slot[0];
#pragma unroll
    for (int i = 0; i + 1 < kStages; i++) slot[i] = slot[i + 1];
    slot[kStages - 1] = t;
  };

  // prologue (scales of the first group(s), K-tiles 0 .. STAGES - 1) and the K loop
  auto run = [&]<bool LA>() __attribute__((always_inline)) {
    constexpr int NL = LA ? 6 : 3;
    load_scales(0);
    if (E) load_scales(1);
#pragma unroll
    for (int t = 0; t < kStages; t++) load_tile.template operator()<LA>(t, t);
    wait_vmcnt<NL * (STAGES - 1)>();
    barrier();
    read_tile.template operator()<0>(0);
    read_scales(0);
    wait_lds_reads();
    take_scales();
    wait_vmcnt<NL * (STAGES - 2)>();
    barrier();  // K-tile 1 is in place, and every wave has K-tile 0 in registers: its slot is free
    int k = 0;
    for (; k + 4 <= nkt; k += 4) {
      step.template operator()<0, LA>(k);
      step.template operator()<1, LA>(k + 1);
      step.template operator()<2, LA>(k + 2);
      step.template operator()<3, LA>(k + 3);
    }
    // a last group of fewer than four K-tiles (K % 512 != 0): the same steps; their loads lie past the end and fetch nothing
    if (k < nkt) step.template operator()<0, LA>(k);
    if (k + 1 < nkt) step.template operator()<1, LA>(k + 1);
    if (k + 2 < nkt) step.template operator()<2, LA>(k + 2);
  };
  if constexpr (WN == 2) {
    run.template operator()<true>();
  } else {
    if (loads_a) run.template operator()<true>();
    else run.template operator()<false>();
  }
  wait_vmcnt<0>();  // no direct load may still be on its way into LDS when the workgroup gives the memory back

  // ---- epilogue, straight from the accumulators.  Register v of lane l is C[m][n] with m = l % 32 and
  // n = 8 (v / 4) + 4 (l / 32) + v % 4 inside a 32 x 32 tile.  bf16: after the conversion lanes l and l + 32 trade halves
  // (v_permlane32_swap), so that every lane owns 8 consecutive outputs and stores them as 16 bytes.
  const int N = args.N, N2 = N * (int)sizeof(OutT);
  const bool edge = rows_a != kBM || rows_b != kBN;
  if constexpr (FUSED) {
    // y = act(acc * row_scale[m] * col_scale[n] + bias[n]) in fp32.  Per 32 x 32 tile a lane owns row 32 i + lane % 32 of its
    // wave's rows and columns 8 q + 4 h .. + 3 for q = 0 .. 3; N % 8 == 0, so a run of four is inside or outside N as a whole
    const void* bias = args.ep.bias;
    const float *row_scale = args.ep.row_scale, *col_scale = args.ep.col_scale;
    const int act = args.ep.act, bias_bf16 = args.ep.bias_bf16;
    const long m0 = (long)pm * kBM + wm * 64 + r32, n0 = (long)pn * kBN + wn * 64 + 4 * h;
    float rs[2];
#pragma unroll
    for (int i = 0; i < 2; i++) rs[i] = row_scale && m0 + i * 32 < args.M ? row_scale[m0 + i * 32] : 1.f;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      if (bias || row_scale || col_scale) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const long n = n0 + j * 32 + q * 8;
          v4f cs = {1.f, 1.f, 1.f, 1.f}, bi = {0.f, 0.f, 0.f, 0.f};
          if (n < N) {
            if (col_scale) cs = *reinterpret_cast<const v4f*>(col_scale + n);
            if (bias && bias_bf16) {
              const u32x2 b2 = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(bias) + n);
              bi = v4f{__uint_as_float(b2[0] << 16), __uint_as_float(b2[0] & 0xffff0000u), __uint_as_float(b2[1] << 16), __uint_as_float(b2[1] & 0xffff0000u)};
            } else if (bias) {
              bi = *reinterpret_cast<const v4f*>(reinterpret_cast<const float*>(bias) + n);
            }
          }
#pragma unroll
          for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][4 * q + e] = fmaf(acc[i][j][4 * q + e] * rs[i], cs[e], bi[e]);
        }
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][j][e] = epilogue_act(acc[i][j][e], act);
    }
  }
  const __amdgpu_buffer_rsrc_t rC = make_rsrc((OutT*)args.C + (size_t)share * args.M * N + (size_t)pm * kBM * N + (size_t)pn * kBN,
                                              (uint32_t)((rows_a - 1) * N + rows_b) * (uint32_t)sizeof(OutT));
  const int row_l = wm * 64 + r32;
  if constexpr (sizeof(OutT) == 2) {
    const int col_l = wn * 64 + 8 * h;
    const int voff = row_l * N2 + col_l * 2;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      uint32_t pk[2][8];
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) pk[j][e] = pack_bf16x2(acc[i][j][2 * e], acc[i][j][2 * e + 1]);
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int c = 0; c < 2; c++) {
            // runs 2t and 2t+1 (dwords 4t+c and 4t+2+c): lower lanes keep run 2t and get the partner's, upper lanes run 2t+1
            const auto x = __builtin_amdgcn_permlane32_swap(pk[j][4 * t + c], pk[j][4 * t + 2 + c], false, false);
            pk[j][4 * t + c] = x[0], pk[j][4 * t + 2 + c] = x[1];
          }
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const v4i v = {(int)pk[j][4 * t], (int)pk[j][4 * t + 1], (int)pk[j][4 * t + 2], (int)pk[j][4 * t + 3]};
          if (!edge || (row_l + i * 32 < rows_a && col_l + j * 32 + t * 16 < rows_b))
            __builtin_amdgcn_raw_buffer_store_b128(v, rC, voff + j * 64 + t * 32, i * 32 * N2, 0);
        }
    }
  } else {
    const int col_l = wn * 64 + 4 * h;
    const int voff = row_l * N2 + col_l * 4;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int gq = 0; gq < 4; gq++) {
          const v4f f = {acc[i][j][4 * gq], acc[i][j][4 * gq + 1], acc[i][j][4 * gq + 2], acc[i][j][4 * gq + 3]};
          if (!edge || (row_l + i * 32 < rows_a && col_l + j * 32 + gq * 8 < rows_b))
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, f), rC, voff + j * 128 + gq * 32, i * 32 * N2, 0);
        }
  }
}

int cu_count_of_device() {
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

// Ring depth: six slots (one workgroup per CU) while the tiles fill at most five eighths of the CUs -- a workgroup is alone
// on its CU anyway, and loads that run six K-tiles ahead cover the way from HBM (256 x 8192 x 8192: 23.0 us against 24.7,
// 1024 x 2048 x 8192: 23.5 against 25.1); three slots beyond, where two workgroups may share a CU and one's waits are the
// other's work (256 tiles: 1024 x 4096 x 4096 18.6 against 20.0, 512 x 8192 x 2048 11.9 against 13.6, 2048 x 2048 x 8192
// 28.8 against 31.2) -- except with K from 6144 on while a CU is left over (512 x 6144 x 16384: six slots 46.0 against
// 51.9, 64 x 28672 x 8192: 34.9 against 38.2, 1 x 27136 x 7680: 30.5 against 34.1; at K = 5120 three: 96 x 20480 x 5120 22.5 against 23.6; between the two six with one row of tiles, 1 x 25600 x 5632 21.2 against 24.6, 32 x 20608 x 5632 19.8 against 22.6, three with more, 512 x 7552 x 5504 23.9 against 24.9), and three slots for K up to 2048, where filling six takes a good part of
// the 8 - 16 K-tiles there are (384 x 2048 x 1024: 6.3 against 7.2, 512 x 4096 x 2048: 10.2 against 11.1, 24 shapes of 384 -
// 1024 rows x N = 2048 .. 6144 all 7 - 14 % ahead).  stages = 3 or 6 forces one (measurement).
template <int FA, int FB, bool FUSED>
hipError_t launch(const GemmArgs& g, const BlockArgs& a, int tiles, int stages, hipStream_t s) {
  const int cus = cu_count_of_device();
  const bool f32 = g.f32out || a.nsplit > 1;  // shares leave fp32 partial sums
  const int grid = tiles * a.nsplit;
  if (g.tile_cols == 256) {  // tiles of 128 x 256, eight waves, four slots
    if (f32) gemm_block_kernel<FA, FB, OutF32, 4, 4, FUSED><<<grid, 512, 0, s>>>(a);
    else gemm_block_kernel<FA, FB, OutBf16, 4, 4, FUSED><<<grid, 512, 0, s>>>(a);
    return hipGetLastError();
  }
  if (stages == 0) stages = ((long)grid * 8 <= (long)cus * 5 && g.K > 2048) || ((g.K >= 6144 || (g.K > 5120 && a.tiles_m == 1) || a.nsplit > 1) && grid < cus) ? 6 : 3;
  if (stages == 6) {
    if (f32) gemm_block_kernel<FA, FB, OutF32, 6, 2, FUSED><<<grid, 256, 0, s>>>(a);
    else gemm_block_kernel<FA, FB, OutBf16, 6, 2, FUSED><<<grid, 256, 0, s>>>(a);
  } else {
    if (f32) gemm_block_kernel<FA, FB, OutF32, 3, 2, FUSED><<<grid, 256, 0, s>>>(a);
    else gemm_block_kernel<FA, FB, OutBf16, 3, 2, FUSED><<<grid, 256, 0, s>>>(a);
  }
  return hipGetLastError();
}
template <int FA, int FB>
hipError_t launch(const GemmArgs& g, const BlockArgs& a, int tiles, int stages, hipStream_t s) {
  // a split leaves the epilogue to the reduction
  if (a.nsplit == 1 && epilogue_any(g.ep)) return launch<FA, FB, true>(g, a, tiles, stages, s);
  return launch<FA, FB, false>(g, a, tiles, stages, s);
}

}  // namespace

bool gemm_block_supports(const GemmArgs& g) {
  // N % 8 keeps every run of 8 bf16 outputs whole and aligned; K in whole K-tiles; 32-bit byte offsets
  // inside one tile's operand rows and inside one tile's rows of C
  return g.M > 0 && g.N > 0 && g.K >= 128 && g.N % 8 == 0 && g.K % 128 == 0 && (long)128 * (g.K / 4 * 3) < (1L << 31) &&
         (long)128 * g.N * 4 < (1L << 31) && (long)((g.M + 127) / 128) <= 65535 && (long)((g.N + 127) / 128) <= 32767 &&
         (long)((g.M + 127) / 128) * ((g.N + 127) / 128) < (1L << 31) && ((uintptr_t)g.C % 16) == 0 && operands_aligned16(g) && !g.fmt_c &&
         !g.no_alloc;
}

// g.ksplit > 1 (with g.ks_part): the K range of every output tile split between that many workgroups, then
// ksplit_reduce_kernel (gemm_tiled.hip), which also applies a fused epilogue.  The caller has checked that the last share
// is not empty (block_split_shares, dispatch.hip).
hipError_t launch_gemm_block(const GemmArgs& g, hipStream_t s) {
  const int bn = g.tile_cols == 256 ? 256 : 128, nsplit = g.ksplit > 1 ? g.ksplit : 1;
  BlockArgs a{g.A, g.B, g.As, g.Bs, nsplit > 1 ? (void*)g.ks_part : g.C, g.M, g.N, g.K, (g.M + kBM - 1) / kBM, (g.N + bn - 1) / bn, g.layout_a, g.layout_b,
              g.raster_group_m > 0 ? g.raster_group_m : kGroupM, g.raster_no_xcd_remap == 1 ? 0 : g.raster_no_xcd_remap == 2 ? 2 : 1, nsplit, g.ep};
  const int tiles = a.tiles_m * a.tiles_n, stages = g.tile_rows == 3 || g.tile_rows == 6 ? g.tile_rows : 0;
  hipError_t e;
  if (g.fmt_a == 2 && g.fmt_b == 2) e = launch<2, 2>(g, a, tiles, stages, s);
  else if (g.fmt_a == 2 && g.fmt_b == 3) e = launch<2, 3>(g, a, tiles, stages, s);
  else if (g.fmt_a == 3 && g.fmt_b == 2) e = launch<3, 2>(g, a, tiles, stages, s);
  else e = launch<3, 3>(g, a, tiles, stages, s);
  if (e == hipSuccess && nsplit > 1) e = launch_ksplit_reduce(g, s);
  return e;
}

}  // namespace mxfp6
