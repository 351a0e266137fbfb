// Mid-M MXFP6 GEMM for gfx950: 32 < M <= 512, where a 256x256 tiling leaves most CUs idle and the
// problem is bound by streaming B (weights) once from HBM and A many times from L2.
//
// One workgroup (8 waves) owns BM rows of A (64 or 128) x BN rows of B (32 or 64) over all of K.  All waves work
// on the same K-tile; operands are staged through LDS by direct loads with the lane->address map and LDS image of
// the tiled kernel (gemm_tiled.hip), in two rings:
//   A ring: three slots of BM rows x 2 K-tiles (192 contiguous bytes per row and slot), from L2;
//   B ring: KB slots of BN rows x GB K-tiles = 24 KB (GB = 256 / BN: 768 or 384 contiguous bytes per row; whole
//           3 KB tiles when B is tile-major), KB - 1 of them in flight: HBM latency is hidden by bytes in flight,
//           and LDS is what limits them (BM = 64: KB = 4, 72 KB in flight; BM = 128: KB = 3, 48 KB).
// Every workgroup re-reads its rows of A from L2, which is what bounds the kernel (about 10.5 TB/s of L2 -> LDS
// traffic in aggregate): BN = 64 halves that traffic per output and is used when N still gives enough workgroups.
// The VMEM counter is in-order, so a wave that waits for a young A slot would also wait for every older B
// slot.  The two streams therefore belong to different waves: waves 0-3 issue all loads of A and of the scales,
// waves 4-7 all loads of B, and each wave waits only for its own stream before the barrier that publishes a slot.
// The E8M0 bytes of eight K-tiles (32 bytes per row) are direct-loaded into one of two small LDS buffers at
// every eighth K-tile, eight K-tiles ahead.  The (BM/32) x (BN/32) accumulator tiles are at most 8, so
// KP = 8 / tiles waves share one 32x32 tile and split the 64-element MFMA steps of K between them; the partial
// tiles are summed through LDS at the end (no scratch, no atomics).
//
// The reference has no kernel for these shapes (its GEMMs need M, N multiples of the 256 tile,
// analysis/bf16_gemm/mi325x/kernel_8192.cpp:24-32).
#include "common.hpp"
#include "kernels.hpp"
#include "loader.hpp"

namespace mxfp6 {

namespace {

constexpr int kBSlot = 24576;  // bytes of one B slot: BN rows x GB K-tiles
constexpr int kASlots = 3;

// wait until at most n of this wave's loads are outstanding (n is one of the sums that occur: see the callers)
#define MXFP6_MID_WAIT(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
__device__ __forceinline__ void wait_loads_md(int n) {
  switch (n) {
    MXFP6_MID_WAIT(1) MXFP6_MID_WAIT(2) MXFP6_MID_WAIT(3) MXFP6_MID_WAIT(4) MXFP6_MID_WAIT(5) MXFP6_MID_WAIT(6)
    MXFP6_MID_WAIT(7) MXFP6_MID_WAIT(8) MXFP6_MID_WAIT(12)
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}
#undef MXFP6_MID_WAIT
__device__ __forceinline__ void barrier_md() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

}  // namespace

template <int FA, int FB, typename Out, int BM, int BN>
__global__ __launch_bounds__(512) void gemm_mid_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                       const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bs,
                                                       typename Out::type* __restrict__ C, int M, int N, int K, int mblocks,
                                                       int layout_b, const Epilogue ep) {
  static_assert((BM == 64 || BM == 128) && (BN == 32 || BN == 64), "tile");
  constexpr int GA = 2;                       // K-tiles per A slot
  constexpr int GB = 256 / BN;                // K-tiles per B slot: 8 or 4
  constexpr int TMW = BM / 32, TNW = BN / 32; // 32-row tiles of A and of B per workgroup
  constexpr int TILES = TMW * TNW;            // accumulator tiles: 2, 4 or 8
  constexpr int KP = 8 / TILES;               // waves per accumulator tile
  constexpr int kASlot = BM * GA * 96;        // 12 or 24 KB
  constexpr int NA = kASlot / 1024 / 4;       // direct loads per A slot and A-wave: 3 or 6
  constexpr int NB = kBSlot / 1024 / 4;       // direct loads per B slot and B-wave: 6
  constexpr int KB = BM == 64 ? 4 : 3;        // B slots
  constexpr int kBRing = kASlots * kASlot;    // B ring starts after the A ring
  constexpr int kScBase = kBRing + KB * kBSlot;
  constexpr int kScBuf = (BM + BN) * 32;      // scales of eight K-tiles: A rows x 32 bytes, then B rows x 32 bytes
  constexpr int kLds = kScBase + 2 * kScBuf;
  static_assert(kLds <= 163840 && kASlots * kASlot >= 8 * 16 * 64 * 4, "LDS budget (the A ring doubles as the reduction buffer)");
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kLds];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int tile = wave % TILES, ti = tile % TMW, tj = tile / TMW;  // accumulator tile of this wave ...
  const int part = wave / TILES;                                     // ... and which MFMA steps of it the wave takes
  const bool a_wave = wave < 4;                  // waves 0-3 load A and the scales, waves 4-7 load B
  const int lw = wave & 3;
  const int nkt = K / 128, sbytes = K / 32, rowbytes = K / 4 * 3, nk4 = nkt / 4;
  // The mblocks workgroups that share rows of B are 8 apart in launch order: workgroups go round-robin over the 8 XCDs,
  // so these land on one XCD at about the same time and the later ones find B in that XCD's L2.  (The last, incomplete
  // group of 8 * mblocks workgroups is numbered consecutively.)
  const int chunk = 8 * mblocks, bid = blockIdx.x, full = (int)(gridDim.x / chunk) * chunk;
  const int nb = bid < full ? (bid / chunk) * 8 + (bid & 7) : bid / mblocks;
  const int mb = bid < full ? (bid % chunk) >> 3 : bid % mblocks;
  const int n0 = nb * BN, m0 = mb * BM;
  const int nrows = min(BN, N - n0), mrows = min(BM, M - m0);

  // rows that do not exist lie past the end of the resource and read as zeros
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A + (size_t)m0 * rowbytes, (uint32_t)mrows * rowbytes);
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(B + (size_t)n0 * rowbytes, (uint32_t)nrows * rowbytes);
  const __amdgpu_buffer_rsrc_t rAs = make_rsrc(As + (size_t)m0 * sbytes, (uint32_t)mrows * sbytes);
  const __amdgpu_buffer_rsrc_t rBs = layout_b ? make_rsrc(Bs + (size_t)nb * TNW * nk4 * 512, (uint32_t)TNW * nk4 * 512)
                                              : make_rsrc(Bs + (size_t)n0 * sbytes, (uint32_t)nrows * sbytes);

  // direct-load address maps.  Load q of a slot fills its LDS bytes [q*1024, q*1024 + 1024); a slot is a sequence of
  // K-tile images (rows x 96 bytes, piece c of row r at r*96 + (c ^ ((r>>3)&1))*16).  A-wave lw takes loads
  // lw*NA .. lw*NA + NA-1 of an A slot, B-wave lw loads lw*NB .. lw*NB + NB-1 of a B slot.
  int voff_ld[NB];  // A-waves use the first NA entries
#pragma unroll
  for (int i = 0; i < NB; i++) {
    if (a_wave) {
      const int o = (lw * NA + (i < NA ? i : 0)) * 64 + lane;
      const int kin = o / (BM * 6), rem = o - kin * (BM * 6), r = rem / 6, c = (rem - r * 6) ^ ((r >> 3) & 1);
      voff_ld[i] = r * rowbytes + kin * 96 + c * 16;
    } else {
      const int o = (lw * NB + i) * 64 + lane;
      const int kin = o / (BN * 6), rem = o - kin * (BN * 6), r = rem / 6, c = (rem - r * 6) ^ ((r >> 3) & 1);
      // tile-major B: K-tile image kin of the slot = the 3 KB tiles (row-tile q, K-tile) of the workgroup's TNW row-tiles
      voff_ld[i] = layout_b ? ((rem / 192) * nkt + kin) * 3072 + (rem % 192) * 16 : r * rowbytes + kin * 96 + c * 16;
    }
  }
  const int bstep = layout_b ? GB * 3072 : GB * 96;  // bytes between B slots

  // scale loads (A-waves): job i < TMW fetches rows 32i .. 32i+31 of A, job TMW + q the rows of B's row-tile q: two lanes
  // per row, 16 bytes (four K-tiles) each; job i belongs to wave i % 4.  LDS image per job: [row][32 bytes]; tile-major
  // scales (two consecutive 512-byte chunks): [half][row][16].
  constexpr int kScJobs = TMW + TNW;
  int n_sc = 0;  // scale loads of this wave per group of eight K-tiles
#pragma unroll
  for (int i = 0; i < kScJobs; i++) n_sc += (a_wave && (i & 3) == wave) ? 1 : 0;
  const int voff_srow = (lane >> 1) * sbytes + (lane & 1) * 16;
  const int sstep_b = layout_b ? 1024 : 32;  // bytes between groups of eight K-tiles
  const int sa_rd = kScBase + (ti * 32 + r32) * 32 + 2 * h;
  const int sb_rd = kScBase + BM * 32 + tj * 1024 + (layout_b ? r32 * 16 : r32 * 32) + 2 * h;
  const int sb_half = layout_b ? 512 : 16;  // offset of K-tiles 4..7 of a group inside B's scale image

  const int sw = (r32 >> 3) & 1;
  int a_rd[3], b_rd[3];
#pragma unroll
  for (int c = 0; c < 3; c++) {
    a_rd[c] = (ti * 32 + r32) * 96 + ((3 * h + c) ^ sw) * 16;
    b_rd[c] = kBRing + (tj * 32 + r32) * 96 + ((3 * h + c) ^ sw) * 16;
  }

  auto issue_scales = [&](int sg) __attribute__((always_inline)) {  // K-tiles 8 sg .. 8 sg + 7 into buffer sg & 1
    const uint32_t dst = lds0 + kScBase + (sg & 1) * kScBuf;
#pragma unroll
    for (int i = 0; i < kScJobs; i++) {
      if (a_wave && (i & 3) == wave) {
        if (i < TMW) {
          dma16(rAs, dst + i * 1024, i * 32 * sbytes + voff_srow, __builtin_amdgcn_readfirstlane(sg * 32));
        } else {
          const int q = i - TMW;
          dma16(rBs, dst + BM * 32 + q * 1024, layout_b ? q * nk4 * 512 + lane * 16 : q * 32 * sbytes + voff_srow,
                   __builtin_amdgcn_readfirstlane(sg * sstep_b));
        }
      }
    }
  };
  auto issue_a = [&](int j) __attribute__((always_inline)) {  // A slot j: K-tiles j*GA .. j*GA + GA-1 (A-waves)
    const uint32_t dst = lds0 + (j % kASlots) * kASlot + lw * (NA * 1024);
    const int so = __builtin_amdgcn_readfirstlane(j * GA * 96);
#pragma unroll
    for (int i = 0; i < NA; i++) dma16(rA, dst + i * 1024, voff_ld[i], so);
  };
  auto issue_b = [&](int b) __attribute__((always_inline)) {  // B slot b: K-tiles GB b .. GB b + GB-1 (B-waves)
    const uint32_t dst = lds0 + kBRing + (b % KB) * kBSlot + lw * (NB * 1024);
    const int so = __builtin_amdgcn_readfirstlane(b * bstep);
#pragma unroll
    for (int i = 0; i < NB; i++) dma16(rB, dst + i * 1024, voff_ld[i], so);
  };

  v16f acc;
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.f;

  const int nslots_a = nkt / GA, nslots_b = nkt / GB, ngroups = nkt / 8;
  // prologue.  A-waves: scales of the first eight K-tiles, A slots 0 and 1.  B-waves: B slots 0 .. KB-2.
  if (a_wave) {
    issue_scales(0);
    issue_a(0);
    if (nslots_a > 1) issue_a(1);
  } else {
#pragma unroll
    for (int b = 0; b < KB - 1; b++)
      if (b < nslots_b) issue_b(b);
  }
  // A-wave loads issued at the boundary in front of K-tile kt, in this order: when kt % 8 == 0 the scales of K-tiles
  // kt + 8 .. kt + 15; always A slot kt/GA + 2
  auto a_issued_at = [&](int kt) __attribute__((always_inline)) -> int {
    int n = 0;
    if ((kt & 7) == 0 && (kt >> 3) + 1 < ngroups) n += n_sc;
    if (kt / GA + 2 < nslots_a) n += NA;
    return n;
  };

  for (int kt0 = 0; kt0 < nkt; kt0 += 8) {
    const int grp = kt0 >> 3;
#pragma unroll
    for (int u = 0; u < 8; u += GA) {
      const int kt = kt0 + u, j = kt / GA, b = kt / GB;
      const bool b_boundary = u % GB == 0;
      // boundary in front of K-tile kt.  A-waves: everything they issued before the previous boundary has landed (A slot j
      // and, at kt % 8 == 0, the scales of this group among it); the previous boundary's loads may stay in flight.
      // B-waves (B-slot boundaries only): B slot b has landed; the slots after it that exist may stay in flight.
      if (a_wave) {
        wait_loads_md(kt == 0 ? (nslots_a > 1 ? NA : 0) : a_issued_at(kt - GA));
      } else if (b_boundary) {
        wait_loads_md(NB * min(KB - 2, nslots_b - 1 - b));
      }
      barrier_md();
      if (a_wave) {
        if (u == 0 && grp + 1 < ngroups) issue_scales(grp + 1);
        if (j + 2 < nslots_a) issue_a(j + 2);
      } else if (b_boundary && b + KB - 1 < nslots_b) {
        issue_b(b + KB - 1);
      }
#pragma unroll
      for (int v = 0; v < GA; v++) {
        const int uu = u + v;  // K-tile kt0 + uu
        // which MFMA steps (64 elements of K) of this K-tile are this wave's: KP = 1: both; KP = 2: step `part`; KP = 4:
        // waves with part < 2 take the even K-tiles, the others the odd ones, step part & 1
        const bool active = KP <= 2 || ((uu & 1) == (part >> 1));
        if (active) {
          const uint8_t* sta = smem + (j % kASlots) * kASlot + v * (BM * 96);
          const uint8_t* stb = smem + (b % KB) * kBSlot + (uu % GB) * (BN * 96);
          const uint8_t* scp = smem + (grp & 1) * kScBuf;
          v4i fa[3], fb[3];
#pragma unroll
          for (int c = 0; c < 3; c++) {
            fb[c] = *reinterpret_cast<const v4i*>(stb + b_rd[c]);
            fa[c] = *reinterpret_cast<const v4i*>(sta + a_rd[c]);
          }
          const int sa = *reinterpret_cast<const uint16_t*>(scp + sa_rd + (uu >> 2) * 16 + (uu & 3) * 4);
          const int sb = *reinterpret_cast<const uint16_t*>(scp + sb_rd + (uu >> 2) * sb_half + (uu & 3) * 4);
          const int step = KP == 2 ? part : (part & 1);
          if (KP == 1 || step == 0) {
            const v8i b0 = __builtin_shufflevector(fb[0], fb[1], 0, 1, 2, 3, 4, 5, -1, -1);
            const v8i a0 = __builtin_shufflevector(fa[0], fa[1], 0, 1, 2, 3, 4, 5, -1, -1);
            acc = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc, sb, sa);
          }
          if (KP == 1 || step == 1) {
            const v8i b1 = __builtin_shufflevector(fb[1], fb[2], 2, 3, 4, 5, 6, 7, -1, -1);
            const v8i a1 = __builtin_shufflevector(fa[1], fa[2], 2, 3, 4, 5, 6, 7, -1, -1);
            acc = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc, sb, sa);
          }
        }
      }
    }
  }

  // sum the KP partial tiles: register e of lane l is C[m = l % 32][n = 8*(e/4) + 4*(l/32) + e%4] of tile (ti, tj).
  // The A ring doubles as the reduction buffer once every wave is past its last LDS read.
  __syncthreads();
  float* partial = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int e = 0; e < 16; e++) partial[(wave * 16 + e) * 64 + lane] = acc[e];
  __syncthreads();
  const bool has_ep = epilogue_any(ep);
  for (int idx = tid; idx < TILES * 1024; idx += 512) {
    const int t = idx >> 10, e = (idx >> 6) & 15, l = idx & 63;
    float s = 0.f;
#pragma unroll
    for (int p = 0; p < KP; p++) s += partial[((p * TILES + t) * 16 + e) * 64 + l];
    const int m = m0 + (t % TMW) * 32 + (l & 31);
    const long nn = (long)n0 + (t / TMW) * 32 + 8 * (e >> 2) + 4 * (l >> 5) + (e & 3);
    if (m < M && nn < N) store1(C + (long)m * N + nn, has_ep ? epilogue_apply(ep, s, m, nn) : s);
  }
}

bool gemm_mid_supports(const GemmArgs& g) {
  // B slots are 8 K-tiles; A row-major (M need not be a multiple of 32)
  if (g.layout_a != 0 || g.M <= 32 || g.M > 512 || g.N <= 0 || g.K < 1024 || g.K % 1024 != 0 || !operands_aligned16(g)) return false;
  if ((long)g.M * (g.K / 4 * 3) >= (1L << 31) || (long)32 * (g.K / 4 * 3) >= (1L << 31)) return false;
  return true;
}

// 64 rows of B per workgroup when 32 would need more than one round of workgroups (tile-major B: whole row-tiles only):
// the time per K-tile and round is about the same for both widths, so halving the rounds is what counts
static bool mid_wide(const GemmArgs& g) {
  const long narrow = (long)((g.N + 31) / 32) * (g.M <= 64 ? 1 : (g.M + 127) / 128);
  return narrow > 256 && (!g.layout_b || g.N % 64 == 0) && (long)64 * (g.K / 4 * 3) < (1L << 31);
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  typedef typename Out::type T;
  const bool wide = mid_wide(g);
  const int nblocks = wide ? (g.N + 63) / 64 : (g.N + 31) / 32;
  const int mblocks = g.M <= 64 ? 1 : (g.M + 127) / 128;
#define MXFP6_MID_LAUNCH(BM, BN) \
  gemm_mid_kernel<FA, FB, Out, BM, BN><<<nblocks * mblocks, 512, 0, s>>>(g.A, g.B, g.As, g.Bs, (T*)g.C, g.M, g.N, g.K, mblocks, g.layout_b, g.ep)
  if (g.M <= 64) {
    if (wide) MXFP6_MID_LAUNCH(64, 64); else MXFP6_MID_LAUNCH(64, 32);
  } else {
    if (wide) MXFP6_MID_LAUNCH(128, 64); else MXFP6_MID_LAUNCH(128, 32);
  }
#undef MXFP6_MID_LAUNCH
  return hipGetLastError();
}

hipError_t launch_gemm_mid(const GemmArgs& g, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (g.fmt_a == FA && g.fmt_b == FB) return g.f32out ? launch<FA, FB, OutF32>(g, s) : launch<FA, FB, OutBf16>(g, s);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipErrorInvalidValue;
}

}  // namespace mxfp6
