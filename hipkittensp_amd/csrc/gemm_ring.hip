// Batched-decode MXFP6 GEMM for gfx950: up to a few hundred rows of A against weights that stream from HBM.
//
// What bounds these shapes is how many bytes of B a compute unit keeps in flight and how long each of them waits for
// the slowest: a workgroup that meets at a barrier every K-tile waits for the slowest of all its loads every time, and
// a ring that holds A and B side by side gives B half the memory.  Here
//   * a workgroup is four consumer waves and one loader wave, and owns 32 * TA rows of A x 128 rows of B over one share
//     of K (K is split between workgroups where the output tiles alone would leave compute units idle);
//   * every consumer wave owns 32 rows of B and streams them through two private 12 KB slots (a chunk = four K-tiles =
//     384 contiguous bytes per row, or four whole 3 KB tiles of a tile-major B): it waits for its own loads only
//     (vmcnt), reads a chunk into registers and refills the slot at once, so that 24 KB per wave, 96 KB per compute
//     unit, are in flight nearly all the time.  No byte of B is shared between waves, so no barrier guards it;
//   * A, which all four consumers need and which comes from L2, is fetched by the loader wave into a ring of four 12 KB
//     slots (a sub-chunk = 4, 2 or 1 K-tiles of 32, 64 or 128 rows), up to three sub-chunks ahead.  Slots are handed
//     over through flags in LDS, the reference's ready / done counters
//     (kernels/gemm/bf16fp32/micros/producer_consumer/32x16/micro_09_async.cpp:129-186): the loader publishes a
//     sub-chunk's number once its loads have landed, consumers count themselves out of a slot once their fragments are
//     in registers, and the loader refills a slot when all four have.  A consumer therefore never waits for another
//     consumer's loads of B, only for A, which is ahead of it.
// There is no workgroup-wide barrier after the first one (which publishes the zeroed flags).  Every wait is on waves of
// the same workgroup, which are all resident, and every spin is bounded.
//
// Shares of a K split leave fp32 partial tiles in a workspace and count themselves in at the tile's arrival counter; the
// workgroup that arrives last sums all shares' tiles in share order (whoever it is: the order of the sum is fixed, so the
// result is bit-reproducible), applies the epilogue, writes C and puts the counter back to zero.  Unsplit, the epilogue is
// applied straight from the accumulators.
// LDS images: B and a row-major A sub-chunk as in the skinny kernel (rows of 96 * KT bytes, 16-byte pieces permuted inside
// groups so that a ds_read_b128 phase is conflict-free), tile-major operands as they are stored.
// The reference has no kernel for these shapes (its GEMMs need M, N multiples of the 256 tile,
// analysis/bf16_gemm/mi325x/kernel_8192.cpp:24-32).  Algorithmic bytes per launch: 0.75*K*(M+N) + (K/32)*(M+N) + 2*M*N.
#include "kernels.hpp"
#include "loader.hpp"

namespace mxfp6 {
namespace {

constexpr int kRingNC = 4;                 // consumer waves per workgroup
constexpr int kRingBN = kRingNC * 32;      // rows of B per workgroup
constexpr int kRingMinChunks = 4;          // chunks of four K-tiles a share of K has at least
constexpr int kRingMaxShares = 8;          // shares of K at most (the workgroup that arrives last holds all of a row-tile's partial sums in registers)

struct RingArgs {
  const uint8_t *A, *B, *As, *Bs;
  void* C;       // the output [M, N]
  float* part;   // nsplit > 1: partial tiles, [tile][share][wave][TA][4][64 lanes][4] floats
  int* counters; // nsplit > 1: one arrival counter per tile, zero between launches
  int M, N, K, layout_a, layout_b, col_tiles, m_blocks, nsplit;
  Epilogue ep;
};

template <typename F>
__device__ __forceinline__ void spin_until(F&& cond) {
  // bounded: a wave that never sees its flag gives up after ~0.1 s of polling instead of hanging the GPU
  for (int n = 0; n < (1 << 21) && !cond(); n++) __builtin_amdgcn_s_sleep(1);
}

// TA: 32-row tiles of A per workgroup (1, 2 or 4)
template <int FA, int FB, typename Out, int TA>
__global__ __launch_bounds__((kRingNC + 1) * 64) void gemm_ring_kernel(const RingArgs args) {
  typedef typename Out::type OutT;
  static_assert(TA == 1 || TA == 2 || TA == 4, "tiles of A");
  constexpr int NC = kRingNC, KT = 4;  // K-tiles per chunk
  constexpr int SA = 4, PA = 3;        // slots of the A ring; sub-chunks the loader keeps in flight
  constexpr int kSlot = 32 * 96 * KT;  // 12 KB: 32 rows of B, or of A (a sub-chunk), over one chunk
  constexpr int NL = kSlot / 1024;     // direct loads per slot
  constexpr int AR = 32 * TA;
  constexpr int NAS = AR > 64 ? 2 : 1;     // loads of A's scales per chunk (16 bytes per row, 64 rows per load)
  constexpr int SAS = TA == 1 ? SA : 2;    // slots of A's scales (per chunk)
  constexpr int NLP = NL + NAS;            // loads of the loader per sub-chunk
  static_assert(kSlot == 12288 && (PA - 1) * NLP < 64, "slot size, vmcnt range");
  constexpr int oB = 0, oBs = oB + NC * 2 * kSlot, oA = oBs + NC * 2 * 1024, oAs = oA + SA * kSlot;
  constexpr int oDummy = oAs + SAS * NAS * 1024, oFlag = oDummy + NAS * 1024, kLds = oFlag + 64;
  static_assert(kLds <= 163840, "LDS budget");
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kLds];
  const uint32_t lds0 = lds_address(smem);
  const uint32_t f_ready = lds0 + oFlag, f_done = lds0 + oFlag + 4 * SA;
  int* const last_flag = reinterpret_cast<int*>(smem + oFlag + 8 * SA);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int K = args.K, M = args.M, N = args.N, layout_a = args.layout_a, layout_b = args.layout_b;
  const int rowbytes = K / 4 * 3, sbytes = K / 32, nk4 = K / 512;  // K % 512 == 0

  // workgroup -> (share of K, column tile, block of rows).  The hardware deals workgroups to the eight XCDs round-robin;
  // XCD x gets the x-th eighth of the share-major order, so that the workgroups that read the same rows of B (the blocks
  // of rows of one column tile and share) sit side by side on one XCD and pull them through its L2 once.
  const int tiles = args.col_tiles * args.m_blocks, total = tiles * args.nsplit;
  int l = blockIdx.x;
  if ((total & 7) == 0) l = (l & 7) * (total >> 3) + (l >> 3);
  const int share = l / tiles, tile = l - share * tiles;
  const int ct = tile / args.m_blocks, mb = tile - ct * args.m_blocks;
  const int cps = (nk4 + args.nsplit - 1) / args.nsplit;
  const int c0 = share * cps, nmine = min(nk4, c0 + cps) - c0;  // this share's chunks: [c0, c0 + nmine), at least one
  const int m0 = mb * AR, n0 = ct * kRingBN + (wave < NC ? wave : 0) * 32;

  if (tid < 2 * SA) reinterpret_cast<int*>(smem + oFlag)[tid] = 0;

  // The image of a slot: 32 rows x 384 bytes with the 16-byte pieces of a row permuted inside groups of eight (piece p of
  // row r at r * 384 + (p ^ ((r >> 1) & 7)) * 16: the 16 rows of a ds_read_b128 phase fall into different banks), produced by
  // choosing which global bytes each lane fetches; a tile-major operand arrives as its four 3 KB tiles of the chunk.
  auto swz = [](int p, int r) __attribute__((always_inline)) { return p ^ ((r >> 1) & 7); };
  auto load_offset = [&](int i, int layout) __attribute__((always_inline)) {  // of load i of a slot, bytes from the first row's (row-tile's) chunk
    const int o = i * 64 + lane, r = o / 24, p = swz(o - r * 24, r);
    return layout ? o * 16 : r * rowbytes + p * 16;
  };
  auto read_offset = [&](int u, int c, int layout) __attribute__((always_inline)) {  // K-tile u, piece c of this lane's half of it
    return layout ? u * 3072 + r32 * 96 + ((3 * h + c) ^ ((r32 >> 3) & 1)) * 16 : r32 * (KT * 96) + swz(u * 6 + 3 * h + c, r32) * 16;
  };

  v16f acc[TA];
  if (wave < NC) {
    // ------------------------------------------------------------------ consumer: 32 rows of B, all rows of A
    const int rows_b = max(0, min(32, N - n0));
    // rows past N lie beyond the end of the resource and read as zeros
    const __amdgpu_buffer_rsrc_t rB = layout_b ? make_rsrc_uniform(args.B + (size_t)(n0 >> 5) * 32 * rowbytes, rows_b ? 32u * rowbytes : 0u)
                                               : make_rsrc_uniform(args.B + (size_t)n0 * rowbytes, (uint32_t)rows_b * rowbytes);
    const __amdgpu_buffer_rsrc_t rBs = layout_b ? make_rsrc_uniform(args.Bs + (size_t)(n0 >> 5) * nk4 * 512, rows_b ? (uint32_t)nk4 * 512 : 0u)
                                                : make_rsrc_uniform(args.Bs + (size_t)n0 * sbytes, (uint32_t)rows_b * sbytes);
    int voff_b[NL];
#pragma unroll
    for (int i = 0; i < NL; i++) voff_b[i] = load_offset(i, layout_b);
    const int voff_bs = layout_b ? r32 * 16 : r32 * sbytes;  // both halves of the wave fetch the same 32 rows
    const uint32_t bbuf = lds0 + oB + wave * (2 * kSlot), bsbuf = lds0 + oBs + wave * 2048;
    auto issue_b = [&](int chunk, int par) __attribute__((always_inline)) {
      const uint32_t pb = __builtin_amdgcn_readfirstlane(par);
      dma16(rBs, bsbuf + pb * 1024, voff_bs, __builtin_amdgcn_readfirstlane(layout_b ? chunk * 512 : chunk * 16));
      const int so = __builtin_amdgcn_readfirstlane(layout_b ? chunk * (KT * 3072) : chunk * (KT * 96));
#pragma unroll
      for (int i = 0; i < NL; i++) dma16(rB, bbuf + pb * kSlot + i * 1024, voff_b[i], so);
    };
    issue_b(c0, 0);
    if (nmine > 1) issue_b(c0 + 1, 1);

    int b_rd[KT][3], a_rd[KT][3];
#pragma unroll
    for (int u = 0; u < KT; u++)
#pragma unroll
      for (int c = 0; c < 3; c++) b_rd[u][c] = read_offset(u, c, layout_b), a_rd[u][c] = read_offset(u, c, layout_a);

#pragma unroll
    for (int t = 0; t < TA; t++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[t][e] = 0.f;

    wait_lds_reads();
    barrier();  // the flags are zero

    int q = 0;  // sub-chunk of A (row-tile t of chunk j: q = j * TA + t), counted from this share's first
    for (int j = 0; j < nmine; j++) {
      if (j + 1 < nmine) wait_vmcnt<NL + 1>(); else wait_vmcnt<0>();  // this chunk has landed; the next one may be in flight
      const int par = j & 1;
      const uint8_t* bp = smem + oB + wave * (2 * kSlot) + par * kSlot;
      v4i fb[KT][3];
      const v4i scb = *reinterpret_cast<const v4i*>(smem + oBs + wave * 2048 + par * 1024 + r32 * 16);
#pragma unroll
      for (int u = 0; u < KT; u++)
#pragma unroll
        for (int c = 0; c < 3; c++) fb[u][c] = *reinterpret_cast<const v4i*>(bp + b_rd[u][c]);
      wait_lds_reads();  // the slot is about to be refilled: its reads must have left LDS
      __builtin_amdgcn_sched_barrier(0);
      if (j + 2 < nmine) issue_b(c0 + j + 2, par);
      v4i sca[TA];
#pragma unroll
      for (int t = 0; t < TA; t++, q++) {
        const int slot = q & (SA - 1);
        spin_until([&]() { return lds_flag_load(f_ready + 4 * slot) == q + 1; });
        const uint8_t* ap = smem + oA + slot * kSlot;
        if (t == 0) {
          const uint8_t* sp = smem + oAs + (TA == 1 ? slot : j & 1) * (NAS * 1024);
#pragma unroll
          for (int tt = 0; tt < TA; tt++) sca[tt] = *reinterpret_cast<const v4i*>(sp + (tt * 32 + r32) * 16);
        }
        v4i fa[KT][3];
#pragma unroll
        for (int u = 0; u < KT; u++)
#pragma unroll
          for (int c = 0; c < 3; c++) fa[u][c] = *reinterpret_cast<const v4i*>(ap + a_rd[u][c]);
        wait_lds_reads();
        __builtin_amdgcn_sched_barrier(0);
        lds_flag_add(f_done + 4 * slot, 1);  // this wave is out of the slot
#pragma unroll
        for (int u = 0; u < KT; u++) {
          const int sb = (uint32_t)scb[u] >> (16 * h), sa = (uint32_t)sca[t][u] >> (16 * h);
          const v8i b0 = __builtin_shufflevector(fb[u][0], fb[u][1], 0, 1, 2, 3, 4, 5, -1, -1);
          const v8i b1 = __builtin_shufflevector(fb[u][1], fb[u][2], 2, 3, 4, 5, 6, 7, -1, -1);
          const v8i a0 = __builtin_shufflevector(fa[u][0], fa[u][1], 0, 1, 2, 3, 4, 5, -1, -1);
          const v8i a1 = __builtin_shufflevector(fa[u][1], fa[u][2], 2, 3, 4, 5, 6, 7, -1, -1);
          acc[t] = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc[t], sb, sa);
          acc[t] = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc[t], sb, sa);
        }
      }
    }
  } else {
    // ------------------------------------------------------------------ loader: A's rows m0 .. m0 + AR - 1 and their scales
    const int rows_a = min(AR, M - m0), rt_a = (rows_a + 31) / 32;
    const __amdgpu_buffer_rsrc_t rA = layout_a ? make_rsrc_uniform(args.A + (size_t)(m0 >> 5) * 32 * rowbytes, (uint32_t)rt_a * 32 * rowbytes)
                                               : make_rsrc_uniform(args.A + (size_t)m0 * rowbytes, (uint32_t)rows_a * rowbytes);
    const __amdgpu_buffer_rsrc_t rAs = layout_a ? make_rsrc_uniform(args.As + (size_t)(m0 >> 5) * nk4 * 512, (uint32_t)rt_a * nk4 * 512)
                                                : make_rsrc_uniform(args.As + (size_t)m0 * sbytes, (uint32_t)rows_a * sbytes);
    int voff_a[NL];
#pragma unroll
    for (int i = 0; i < NL; i++) voff_a[i] = load_offset(i, layout_a);
    int voff_as[NAS];
#pragma unroll
    for (int i = 0; i < NAS; i++) {
      const int row = i * 64 + lane;
      voff_as[i] = layout_a ? (row >> 5) * (nk4 * 512) + (row & 31) * 16 : row * sbytes;
    }
    wait_lds_reads();
    barrier();  // the flags are zero

    const int nq = nmine * TA;
    int issued = 0, signalled = 0;
    for (;;) {
      bool can_issue = issued < nq && issued - signalled < PA;
      if (can_issue && issued >= SA) can_issue = lds_flag_load(f_done + 4 * (issued & (SA - 1))) >= NC * (issued / SA);  // all consumers are out of the slot
      if (can_issue) {
        const int j = issued / TA, t = issued - j * TA, slot = issued & (SA - 1), chunk = c0 + j;
        // the chunk's scales ride with its first sub-chunk; the others issue the same loads into a place nobody reads, so
        // that every batch counts the same
        const uint32_t sdst = __builtin_amdgcn_readfirstlane(lds0 + (t == 0 ? oAs + (TA == 1 ? slot : j & 1) * (NAS * 1024) : oDummy));
        const int sos = __builtin_amdgcn_readfirstlane(layout_a ? chunk * 512 : chunk * 16);
#pragma unroll
        for (int i = 0; i < NAS; i++) dma16(rAs, sdst + i * 1024, voff_as[i], sos);
        // the row-tile's offset rides in the per-lane offset, which the hardware checks against the end of the resource
        // (the scalar offset it does not): rows past M read as zeros
        const int tv = t * 32 * rowbytes;
        const int so = __builtin_amdgcn_readfirstlane(layout_a ? chunk * (KT * 3072) : chunk * (KT * 96));
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds0 + oA + slot * kSlot);
#pragma unroll
        for (int i = 0; i < NL; i++) dma16(rA, dst + i * 1024, voff_a[i] + tv, so);
        issued++;
      } else if (signalled < issued) {
        // the oldest batch in flight has landed once at most the younger ones remain
        const int younger = issued - signalled - 1;
        if (younger >= 2) wait_vmcnt<2 * NLP>(); else if (younger == 1) wait_vmcnt<NLP>(); else wait_vmcnt<0>();
        lds_flag_store(f_ready + 4 * (signalled & (SA - 1)), signalled + 1);
        signalled++;
      } else if (issued >= nq) {
        break;
      } else {
        __builtin_amdgcn_s_sleep(1);  // the next slot is still being read and nothing is in flight
      }
    }
  }

  // ---- output.  Register e of lane l of consumer wave w is C[m0 + 32 t + l % 32][n0 + 8 (e / 4) + 4 (l / 32) + e % 4];
  // N % 4 == 0, so a run of four is inside or outside N as a whole.
  if (args.nsplit > 1) {
    // K split: every workgroup leaves its partial tile in the workspace; the one that arrives last (a counter per tile)
    // adds the shares up in share order, so the result does not depend on who that is, and nobody waits for anybody.
    // The other workgroups run on XCDs with L2s of their own: partial tiles and counter are written and read with
    // device-scope atomic accesses, which go past those caches (device-scope fences would write back and invalidate a
    // whole L2 per wave).
    float* const tile_part = args.part + (size_t)tile * args.nsplit * (NC * TA * 1024);
    if (wave < NC) {
      float* mine = tile_part + ((size_t)share * NC + wave) * (TA * 1024);
#pragma unroll
      for (int t = 0; t < TA; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) __hip_atomic_store(mine + (t * 16 + e) * 64 + lane, acc[t][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      wait_vmcnt<0>();  // stores count there too: the partial tile has arrived before the counter moves
    }
    barrier();
    if (tid == 0) *last_flag = __hip_atomic_fetch_add(args.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == args.nsplit - 1;
    __syncthreads();
    if (!*last_flag || wave >= NC) return;
    // all shares' loads of a row-tile go out before the first sum (one round trip to memory, not one per share);
    // the order of summation is share order whoever adds
    const float* mine0 = tile_part + (size_t)wave * (TA * 1024) + lane;
    const size_t share_stride = (size_t)NC * (TA * 1024);
#pragma unroll
    for (int t = 0; t < TA; t++) {
      float v[kRingMaxShares][16];
#pragma unroll
      for (int s = 0; s < kRingMaxShares; s++)
        if (s < args.nsplit) {
#pragma unroll
          for (int e = 0; e < 16; e++) v[s][e] = __hip_atomic_load(mine0 + s * share_stride + (t * 16 + e) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
      for (int e = 0; e < 16; e++) acc[t][e] = v[0][e];
#pragma unroll
      for (int s = 1; s < kRingMaxShares; s++)
        if (s < args.nsplit) {
#pragma unroll
          for (int e = 0; e < 16; e++) acc[t][e] += v[s][e];
        }
    }
    if (tid == 0) __hip_atomic_store(args.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
  } else if (wave >= NC) {
    return;
  }
  const bool has_ep = epilogue_any(args.ep);
#pragma unroll
  for (int t = 0; t < TA; t++) {
    const long m = (long)m0 + 32 * t + r32;
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++) {
      const long n = (long)n0 + 8 * g4 + 4 * h;
      if (m >= M || n >= N) continue;
      float v[4] = {acc[t][4 * g4], acc[t][4 * g4 + 1], acc[t][4 * g4 + 2], acc[t][4 * g4 + 3]};
      if (has_ep) {
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = epilogue_apply(args.ep, v[e], m, n + e);
      }
      store4(reinterpret_cast<OutT*>(args.C) + (size_t)m * N + n, v[0], v[1], v[2], v[3]);
    }
  }
}

int cu_count_ring() {
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

struct RingPlan {
  int ta, m_blocks, col_tiles, nsplit;
};

// Blocks of rows, column tiles and shares of K.  want: 0 = as many shares as leave no compute unit idle (every share at
// least kRingMinChunks chunks of four K-tiles), 1 = none, n = n if K allows
RingPlan ring_plan(const GemmArgs& g, int want) {
  RingPlan p;
  p.ta = g.M <= 32 ? 1 : g.M <= 64 ? 2 : 4;
  p.m_blocks = (g.M + 32 * p.ta - 1) / (32 * p.ta);
  p.col_tiles = (g.N + kRingBN - 1) / kRingBN;
  const int nchunks = g.K / 512;
  const long tiles = (long)p.m_blocks * p.col_tiles;
  int cus = cu_count_ring();
  if (cus <= 0) cus = 256;
  long s = want > 1 ? want : want == 1 ? 1 : cus / tiles;
  if (want <= 0 && s > nchunks / kRingMinChunks) s = nchunks / kRingMinChunks;
  if (s > nchunks) s = nchunks;
  if (s > kRingMaxShares) s = kRingMaxShares;
  if (s < 1) s = 1;
  const int cps = (nchunks + (int)s - 1) / (int)s;
  p.nsplit = (nchunks + cps - 1) / cps;  // no empty share
  return p;
}

}  // namespace

bool gemm_ring_supports(const GemmArgs& g) {
  return g.M >= 1 && g.N >= 4 && g.N % 4 == 0 && g.K >= 512 && g.K % 512 == 0 && (long)128 * (g.K / 4 * 3) < (1L << 31) && !g.fmt_c &&
         ((uintptr_t)g.C % 16) == 0 && operands_aligned16(g) && (long)g.M * g.N < (1L << 40);
}

// K split of this kernel for a call: shares (1 = none), and the bytes of partial tiles and the arrival counters it needs
int ring_ksplit_plan(const GemmArgs& g, int want, size_t* part_bytes, size_t* counters) {
  *part_bytes = 0, *counters = 0;
  if (!gemm_ring_supports(g) || g.no_alloc) return 1;
  const RingPlan p = ring_plan(g, want);
  if (p.nsplit > 1) {
    *counters = (size_t)p.m_blocks * p.col_tiles;
    *part_bytes = *counters * p.nsplit * (kRingNC * p.ta * 1024) * sizeof(float);
  }
  return p.nsplit;
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  const bool split = g.ksplit > 1 && g.ks_part && g.ks_counters;
  RingPlan p = ring_plan(g, split ? g.ksplit : 1);
  if (split && p.nsplit != g.ksplit) return hipErrorInvalidValue;
  RingArgs ra = {g.A, g.B, g.As, g.Bs, g.C, g.ks_part, g.ks_counters, g.M, g.N, g.K, g.layout_a, g.layout_b, p.col_tiles, p.m_blocks, p.nsplit, g.ep};
  const unsigned grid = (unsigned)p.col_tiles * p.m_blocks * p.nsplit;
  constexpr int threads = (kRingNC + 1) * 64;
  if (p.ta == 1) gemm_ring_kernel<FA, FB, Out, 1><<<grid, threads, 0, s>>>(ra);
  else if (p.ta == 2) gemm_ring_kernel<FA, FB, Out, 2><<<grid, threads, 0, s>>>(ra);
  else gemm_ring_kernel<FA, FB, Out, 4><<<grid, threads, 0, s>>>(ra);
  return hipGetLastError();
}

hipError_t launch_gemm_ring(const GemmArgs& g, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (g.fmt_a == FA && g.fmt_b == FB) return g.f32out ? launch<FA, FB, OutF32>(g, s) : launch<FA, FB, OutBf16>(g, s);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipErrorInvalidValue;
}

}  // namespace mxfp6
