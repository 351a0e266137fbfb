// LDS-tiled MXFP6 GEMM for gfx950, 4-wave interleaved variant: 256x256 output tile per workgroup, K-tile 128, one
// wave per SIMD with a 128x128 wave tile (16 accumulators of 32x32 = 256 registers, which the compiler places in
// the accumulation registers) and two fragment sets.  This is the schedule the reference measures against its 8-wave
// ping-pong for the same MFMA family (analysis/paper_experiments/pingpong_micro/plot.py:16-19); it is kept as a
// selectable kernel (mxfp6_set_kernel(18)) so that the choice of schedule rests on counters for both candidates.
// It reads a third fewer bytes from LDS per K-tile than the 8-wave kernel (96 KB against 144 KB) and pays with one
// wave per SIMD: any stall of that wave stalls the SIMD's matrix core.
//
// Every wave runs one software-pipelined stream: during the 32 MFMAs of K-tile p it reads the fragments
// of K-tile p+1 from LDS into the other fragment set and issues its share of the direct-to-LDS loads of
// K-tile p+3 (into the ring slot of K-tile p, which every wave finished reading before the barrier that
// closed phase p-1), three loads per eight MFMAs.  One barrier per K-tile.  LDS image, operand mapping and raster
// are the ones of the 8-wave kernel (gemm_tiled.hip); one workgroup per output tile, bf16 tiles staged through
// LDS for the store; no fused epilogue.
#include "common.hpp"
#include "kernels.hpp"
#include "loader.hpp"

namespace mxfp6 {
namespace t4 {

constexpr int kBM = 256, kBN = 256, kBK = 128;
constexpr int kOpStage = 256 * 96;
constexpr int kScStage = 256 * 16;
constexpr int kGroupM = 4;
constexpr int kStages = 3;
constexpr int kStage = 2 * kOpStage, kScaleBase = kStages * kStage, kScaleBuf = 2 * kScStage;
constexpr int kLdsBytes = kScaleBase + 2 * kScaleBuf;
constexpr int WM = 2, WN = 2, NW = WM * WN;
constexpr int TM = 8 / WM, TN = 8 / WN;
constexpr int OPS = 24 / NW;  // operand direct loads per wave per operand per K-tile
constexpr int SCL = 2;        // scale direct loads per wave per batch that carries scales (one for A, one for B)
constexpr int NMMA = 2 * TM * TN;
static_assert(kLdsBytes <= 163840, "LDS budget");


template <int FA, int FB, typename Out>
__global__ __launch_bounds__(NW * 64) void gemm_tiled4_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                              const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bs,
                                                              typename Out::type* __restrict__ C, int M, int N, int K,
                                                              int tiles_m, int tiles_n, int layout_a, int layout_b) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kLdsBytes];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem;

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
  const int rows_a = min(kBM, M - pm * kBM), rows_b = min(kBN, N - pn * kBN);
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A + (size_t)pm * kBM * rowbytes, (uint32_t)rows_a * rowbytes);
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(B + (size_t)pn * kBN * rowbytes, (uint32_t)rows_b * rowbytes);
  const int nk4 = (nkt + 3) / 4;
  const __amdgpu_buffer_rsrc_t rSA = layout_a ? make_rsrc(As + (size_t)pm * (kBM / 32) * nk4 * 512, (uint32_t)((rows_a + 31) / 32) * nk4 * 512) : make_rsrc(As + (size_t)pm * kBM * sbytes, (uint32_t)rows_a * sbytes);
  const __amdgpu_buffer_rsrc_t rSB = layout_b ? make_rsrc(Bs + (size_t)pn * (kBN / 32) * nk4 * 512, (uint32_t)((rows_b + 31) / 32) * nk4 * 512) : make_rsrc(Bs + (size_t)pn * kBN * sbytes, (uint32_t)rows_b * sbytes);

  // per-lane global byte offsets of the direct loads.  Load q = wave*OPS + n fills LDS bytes [q*1024, q*1024 + 1024)
  // of the operand tile; three consecutive loads cover exactly 32 rows, so load n of a wave differs from load
  // n % 3 by a uniform offset (32 rows, or one row-tile of a tile-major operand) that rides in the scalar offset.
  int voff_a[3], voff_b[3];
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int q = wave * OPS + i, o = q * 64 + lane;
    const int r = o / 6, c = (o - r * 6) ^ ((r >> 3) & 1);
    const int vrow = r * rowbytes + c * 16;
    const int vtile = (q / 3) * (nkt * 3072) + (q % 3) * 1024 + lane * 16;
    voff_a[i] = layout_a ? vtile : vrow;
    voff_b[i] = layout_b ? vtile : vrow;
  }
  const int kstep_a = layout_a ? 3072 : 96, kstep_b = layout_b ? 3072 : 96;
  const int up_a = layout_a ? nkt * 3072 : 32 * rowbytes, up_b = layout_b ? nkt * 3072 : 32 * rowbytes;
  const int srow = wave * 64 + lane;  // wave w fetches the scales of rows 64w .. 64w+63 of A and of B
  const int voff_sa = layout_a ? (srow >> 5) * nk4 * 512 + (srow & 31) * 16 : srow * sbytes;
  const int voff_sb = layout_b ? (srow >> 5) * nk4 * 512 + (srow & 31) * 16 : srow * sbytes;
  const int sstep_a = layout_a ? 512 : 16, sstep_b = layout_b ? 512 : 16;

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

  auto issue_scales = [&](int grp) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + kScaleBase + (grp & 1) * kScaleBuf + wave * 1024;
    // (the group's offset in the per-lane offset: that is the one the hardware checks against the end of the resource)
    dma16(rSA, dst, voff_sa + grp * sstep_a, 0);
    dma16(rSB, dst + kScStage, voff_sb + grp * sstep_b, 0);
  };
  auto issue_one = [&](int t, int slot, int n) __attribute__((always_inline)) {
    const uint32_t dst = lds0 + slot * kStage + wave * (OPS * 1024);
    if (n < OPS) dma16(rA, dst + n * 1024, voff_a[n % 3], t * kstep_a + (n / 3) * up_a);
    else dma16(rB, dst + kOpStage + (n - OPS) * 1024, voff_b[(n - OPS) % 3], t * kstep_b + ((n - OPS) / 3) * up_b);
  };
  auto issue_ops = [&](int t, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int n = 0; n < 2 * OPS; n++) issue_one(t, slot, n);
  };

  // two fragment sets: MFMAs read one while the LDS reads of the next K-tile fill the other
  v12i fa[2][TM], fb[2][TN];
  int sca[2][TM], scb[2][TN];
  // LDS read r (0 .. 3*(TM+TN)-1) of one K-tile: B tiles first, then A tiles, three pieces each
  auto read_one = [&](int buf, int slot, int r) __attribute__((always_inline)) {
    const uint8_t* st = smem + slot * kStage;
    const int t = r / 3, c = r % 3;
    if (t < TN) {
      const v4i p = *reinterpret_cast<const v4i*>(st + b_rd[c] + t * 3072);
#pragma unroll
      for (int e = 0; e < 4; e++) fb[buf][t][4 * c + e] = p[e];
    } else {
      const v4i p = *reinterpret_cast<const v4i*>(st + a_rd[c] + (t - TN) * 3072);
#pragma unroll
      for (int e = 0; e < 4; e++) fa[buf][t - TN][4 * c + e] = p[e];
    }
  };
  // scale read r (0 .. TM+TN-1) of K-tile `tile`
  auto read_scale = [&](int buf, int sc_off, int r) __attribute__((always_inline)) {
    const uint8_t* sc = smem + sc_off;
    if (r < TN) scb[buf][r] = *reinterpret_cast<const uint16_t*>(sc + sb_rd + r * 512);
    else sca[buf][r - TN] = *reinterpret_cast<const uint16_t*>(sc + sa_rd + (r - TN) * 512);
  };
  auto pin = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; i++) asm volatile("" : "+v"(fa[buf][i]));
#pragma unroll
    for (int j = 0; j < TN; j++) asm volatile("" : "+v"(fb[buf][j]));
  };
  auto mma_tile = [&](int buf, auto&& between) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const v8i a0 = __builtin_shufflevector(fa[buf][i], fa[buf][i], 0, 1, 2, 3, 4, 5, -1, -1);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const v8i b0 = __builtin_shufflevector(fb[buf][j], fb[buf][j], 0, 1, 2, 3, 4, 5, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc[i][j], scb[buf][j], sca[buf][i]);
        between(i * TN + j);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const v8i a1 = __builtin_shufflevector(fa[buf][i], fa[buf][i], 6, 7, 8, 9, 10, 11, -1, -1);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const v8i b1 = __builtin_shufflevector(fb[buf][j], fb[buf][j], 6, 7, 8, 9, 10, 11, -1, -1);
        acc[i][j] = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc[i][j], scb[buf][j], sca[buf][i]);
        between(TM * TN + i * TN + j);
      }
    }
  };

  // ---- phase p: MFMAs of tile p (fragment set p & 1), LDS reads of tile p+1, loads of tile p+3.
  // At the end: own LDS reads done, own share of tile p+2 landed (the batch just issued may stay in
  // flight), barrier.  PM = p mod 4; STEADY: tiles p+1 .. p+3 and the scale group the batch carries exist.
  int slot_rd = 1, slot_ld = 0;  // ring slots of tile p+1 and of tile p+3 (= slot of tile p)
  auto phase = [&]<int PM, bool STEADY>(int p) __attribute__((always_inline)) {
    constexpr int BUF = PM & 1, KMR = (PM + 1) & 3;  // KMR: (p+1) mod 4, position of tile p+1 inside its scale group
    const bool has_rd = STEADY || p + 1 < nkt;
    const bool has_ld = STEADY || p + 3 < nkt;
    const bool has_sc = PM == 0 && (STEADY || p + 4 < nkt);
    const int sc_off = (((p + 1) >> 2) & 1) * kScaleBuf + KMR * 4;
    mma_tile(BUF, [&](int i) __attribute__((always_inline)) {
      __builtin_amdgcn_sched_barrier(0);
      if (has_rd) {
        if (i < 3 * (TM + TN)) read_one(BUF ^ 1, slot_rd, i);
        else if (i - 3 * (TM + TN) < TM + TN) read_scale(BUF ^ 1, sc_off, i - 3 * (TM + TN));
      }
      if (has_ld) {
        // 12 loads over 32 MFMA slots: slots 0,3,5 of every 8; the scale loads ride in slots 30 and 31
        if ((i & 7) == 0 || (i & 7) == 3 || (i & 7) == 5) issue_one(p + 3, slot_ld, 3 * (i >> 3) + ((i & 7) == 0 ? 0 : (i & 7) == 3 ? 1 : 2));
        if (i == 31 && has_sc) issue_scales((p + 4) >> 2);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    wait_lds_reads();
    if (has_rd) pin(BUF ^ 1);
    if (has_ld) {
      if (has_sc) wait_vmcnt<2 * OPS + SCL>(); else wait_vmcnt<2 * OPS>();
    } else {
      wait_vmcnt<0>();
    }
    barrier();
    slot_rd = slot_rd == kStages - 1 ? 0 : slot_rd + 1;
    slot_ld = slot_ld == kStages - 1 ? 0 : slot_ld + 1;
  };

  // prologue: scales of the first four K-tiles and tiles 0, 1, 2; tiles 0 and 1 must have landed everywhere
  // before phase 0 (which reads tile 1), and every wave must have read tile 0 before phase 0 refills its slot
  issue_scales(0);
  issue_ops(0, 0);
  if (nkt > 1) issue_ops(1, 1);
  if (nkt > 2) {
    issue_ops(2, 2);
    wait_vmcnt<2 * OPS>();
  } else {
    wait_vmcnt<0>();
  }
  barrier();
#pragma unroll
  for (int r = 0; r < 3 * (TM + TN); r++) read_one(0, 0, r);
#pragma unroll
  for (int r = 0; r < TM + TN; r++) read_scale(0, 0, r);
  wait_lds_reads();
  pin(0);
  barrier();

  {
    int p = 0;
    for (; p + 8 <= nkt; p += 4) {
      phase.template operator()<0, true>(p);
      phase.template operator()<1, true>(p + 1);
      phase.template operator()<2, true>(p + 2);
      phase.template operator()<3, true>(p + 3);
    }
    for (; p < nkt; p += 4) {
      phase.template operator()<0, false>(p);
      if (p + 1 < nkt) phase.template operator()<1, false>(p + 1);
      if (p + 2 < nkt) phase.template operator()<2, false>(p + 2);
      if (p + 3 < nkt) phase.template operator()<3, false>(p + 3);
    }
  }

  if constexpr (sizeof(typename Out::type) == 2) {
    constexpr int kRowPitch = 512 + 16;
    static_assert(256 * kRowPitch <= kLdsBytes, "C tile fits the ring");
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
    const int chunk = tid & 31, row0 = tid >> 5;
    uint8_t* cg = reinterpret_cast<uint8_t*>(C) + ((size_t)pm * kBM + row0) * (size_t)N * 2 + (size_t)pn * kBN * 2 + chunk * 16;
    constexpr int kRowsPerPass = NW * 2;
    const bool col_ok = chunk * 8 < rows_b;
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

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  const int tm = (g.M + kBM - 1) / kBM, tn = (g.N + kBN - 1) / kBN;
  gemm_tiled4_kernel<FA, FB, Out><<<tm * tn, NW * 64, 0, s>>>(g.A, g.B, g.As, g.Bs, (typename Out::type*)g.C, g.M, g.N, g.K, tm, tn,
                                                             g.layout_a, g.layout_b);
  return hipGetLastError();
}

}  // namespace t4

bool gemm_tiled4_supports(const GemmArgs& g) {
  return gemm_tiled_supports(g) && !epilogue_any(g.ep) && !g.fmt_c && (long)g.M * g.N < (1L << 40);
}

hipError_t launch_gemm_tiled4(const GemmArgs& g, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (g.fmt_a == FA && g.fmt_b == FB) return g.f32out ? t4::launch<FA, FB, OutF32>(g, s) : t4::launch<FA, FB, OutBf16>(g, s);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipErrorInvalidValue;
}

}  // namespace mxfp6
