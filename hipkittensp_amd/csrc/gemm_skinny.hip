// Skinny-M (decode-shaped) MXFP6 GEMM for gfx950: M <= 128, bound by HBM.
//
// Every byte of B (weights) is read from HBM once.  One workgroup owns 32 consecutive rows of B (32 output
// columns) and splits K over its waves in chunks of four K-tiles (4 x 128 elements = 384 bytes per row = three
// whole 128-byte lines), dealt round-robin: wave w takes chunks w, w+NW, ... so the workgroup streams one
// contiguous K range of its 32 rows.  Each wave owns a private LDS buffer for one chunk (B: 12 KB, A: 6 or 12 KB)
// and runs
//   issue the chunk's direct loads -> wait for all of them -> LDS -> registers (all four K-tiles) ->
//   issue the next chunk's loads -> 8 MFMAs
// so that a wave's whole buffer is in flight except while it is being read out (a few hundred clocks against
// microseconds of HBM latency), and the 6-8 waves of a workgroup are out of phase with each other.
// A direct load fetches, per row, the chunk's 384 contiguous bytes (24 lanes x 16 bytes), i.e. whole cache lines:
// a row-major B costs the same L2 requests and HBM bursts as a tile-major one.  The LDS image of a row-major
// chunk is [row][384 bytes] with the 16-byte pieces of a row permuted inside groups of eight,
//     piece p of row r lives at  r * 384 + (p ^ ((r >> 1) & 7)) * 16,
// which spreads the 16 rows of a ds_read_b128 phase over all 64 banks (rows r and r+16 share banks and are never
// in the same phase, analysis/paper_experiments/phases/ds_read_b128/phase_results.txt:4-7); the permutation is
// applied by choosing which global bytes each lane fetches, as in the tiled kernel.  A tile-major B arrives as
// four 3 KB tiles in the tiled kernel's image.  A's rows are staged like a row-major B, from L2: 16 or 32 of them
// feed one 32x32 accumulator tile per wave; 64 feed two and 128 four (against the same fragments of B), with four
// waves per workgroup, and 128 in chunks of two K-tiles (192-byte rows), so that the buffers still fit LDS.  The
// E8M0 bytes of a chunk are 16 bytes per row: one more direct load each for B and A (no load of this kernel has a
// register destination, so nothing can read a register before its load has landed).  All loads are issued from
// inline assembly and waited for with vmcnt by hand.  The partial 32x32 tiles of the waves are summed
// through LDS: no scratch, no atomics.
//
// The reference has no kernel for this shape (its GEMMs need M, N multiples of the 256 tile,
// analysis/bf16_gemm/mi325x/kernel_8192.cpp:24-32).  Algorithmic bytes per launch:
// 0.75*K*(M+N) + (K/32)*(M+N) + 2*M*N.
#include <map>
#include <mutex>
#include <utility>
#include "common.hpp"
#include "kernels.hpp"
#include "loader.hpp"

// Scratch memory of mxfp6_gemm_noalloc: kScratchSlots partial tiles of 4 KB (one per (tile, split) pair of a K split) followed by
// kScratchTiles arrival counters.  In host code this name is only a handle for hipGetSymbolAddress; kernels get the device
// address that call returns.
constexpr int kScratchSlots = 256, kScratchTiles = 256;
static __device__ __align__(256) unsigned char scratch[kScratchSlots * 4096 + kScratchTiles * 4];

namespace mxfp6 {

// AR = rows of A staged (16, 32 or 64: one or two 32-row accumulator tiles per wave); NW = waves per workgroup;
// BR = rows of B per workgroup (32; 16 so that a narrow N still gives every CU a workgroup: the MFMA's other 16
// rows then mirror the first and their outputs are dropped; 64 = two 32-row tiles of B against every fragment of A,
// which halves the bytes of A a workgroup pulls from L2 per byte of B)
template <int FA, int FB, typename Out, int AR, int NW, int BR, int DB>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                              const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bs,
                                                              typename Out::type* __restrict__ C, int M, int N, int K, int layout_b,
                                                              const Epilogue ep, int nsplit, float* ws_part, int* ws_cnt) {
  static_assert(BR == 64 || BR == 32 || BR == 16, "rows of B per workgroup");
  static_assert(AR == 16 || AR == 32 || AR == 64 || AR == 128, "rows of A");
  constexpr int TA = AR > 32 ? AR / 32 : 1;   // 32-row tiles of A per wave
  constexpr int TB = BR == 64 ? 2 : 1;        // 32-row tiles of B per wave
  constexpr int TT = TA * TB;                 // accumulator tiles per wave (tile t of A, tb of B: t * TB + tb)
  constexpr int KT = AR == 128 ? 2 : 4;       // K-tiles per chunk (128 rows of A: half chunks, so that four waves' buffers fit)
  constexpr int kRow = 96 * KT, kPieces = 6 * KT;  // bytes and 16-byte pieces of a row in a chunk
  // a wave's buffer: DB chunks of B (DB = 2: the chunk after the next is on its way from HBM while the next one's A, which
  // comes from L2 in a fraction of that time, is fetched one chunk ahead), one chunk of A, then the scales:
  static_assert(DB == 1 || DB == 2, "chunks of B per wave");
  constexpr int kBBuf = BR * kRow, kABuf = AR * kRow, kAOff = DB * kBBuf, kScOff = kAOff + kABuf;
  constexpr int kASc = AR <= 64 ? 1024 : AR * 16;                              // 1 KB per chunk of B, 16 bytes per row of A
  constexpr int kAScOff = kScOff + DB * 1024;
  constexpr int kBuf = kAScOff + kASc;
  constexpr int NBL = kBBuf / 1024, NAL = kABuf / 1024, NAS = kASc / 1024;  // direct loads per chunk: 12 or 6; 6, 12 or 24; 1 or 2
  static_assert(kBBuf % 1024 == 0 && kABuf % 1024 == 0, "whole direct loads");
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NW * kBuf];
  static_assert(NW * kBuf <= 163840 && NW * kBuf >= NW * TT * 16 * 64 * 4 + 64, "LDS budget (the buffers double as the reduction buffer)");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int nkt = K / 128, sbytes = K / 32, rowbytes = K / 4 * 3;
  // nsplit > 1: the K range is split between nsplit workgroups per BR rows of B (workgroup = split * ntiles + tile)
  const int ntiles = gridDim.x / nsplit;
  const int tile = blockIdx.x % ntiles, split = blockIdx.x / ntiles;
  const int n0 = tile * BR;
  const int nrows = min(BR, N - n0);
  // tile-major B: first row-tile of this workgroup, how many it has, and (BR = 16) which 16 rows of it
  const int rt = BR == 64 ? tile * 2 : BR == 32 ? tile : tile >> 1, half = BR == 16 ? tile & 1 : 0;
  const int nrt = BR == 64 ? min(2, (N + 31) / 32 - rt) : 1;

  // rows that do not exist (n >= N, m >= M) lie past the end of the resource and read as zeros
  const __amdgpu_buffer_rsrc_t rB = layout_b ? make_rsrc(B + (size_t)rt * 32 * rowbytes, (uint32_t)nrt * 32 * rowbytes)
                                             : make_rsrc(B + (size_t)n0 * rowbytes, (uint32_t)nrows * rowbytes);
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A, (uint32_t)M * rowbytes);
  // tile-major B: this workgroup's 32 rows are one row-tile, whose scales are nk4 chunks of 512 bytes (row r at r * 16)
  const int nk4 = nkt / 4;
  const __amdgpu_buffer_rsrc_t rBs = layout_b ? make_rsrc(Bs + (size_t)rt * nk4 * 512, (uint32_t)nrt * nk4 * 512)
                                              : make_rsrc(Bs + (size_t)n0 * sbytes, (uint32_t)nrows * sbytes);
  const __amdgpu_buffer_rsrc_t rAs = make_rsrc(As, (uint32_t)M * sbytes);

  // direct-load address maps: load i fills LDS bytes [i*1024, i*1024 + 1024) of the buffer; slot o = i*64 + lane holds
  // piece swz(o % kPieces, row) of row o / kPieces, where swz permutes the pieces of a row inside groups of eight
  // (384-byte rows) or four (192-byte rows) so that the 16 rows of a ds_read_b128 phase fall into different banks.
  // Tile-major B: KT consecutive 3 KB tiles, copied as they are (BR = 16: the 1536 bytes that this workgroup's 16 rows
  // have in each of them).
  auto swz = [](int p, int r) __attribute__((always_inline)) { return KT == 4 ? p ^ ((r >> 1) & 7) : p ^ ((r >> 2) & 3); };
  int voff_b[NBL], voff_a[NAL];
#pragma unroll
  for (int i = 0; i < NBL; i++) {
    const int o = i * 64 + lane, r = o / kPieces, p = swz(o - r * kPieces, r);
    constexpr int kPer = (BR == 16 ? 16 : 32) * 6;  // 16-byte pieces per K-tile of one row-tile (BR = 16: of this workgroup's half of it)
    constexpr int kPerRt = KT * kPer;                // ... per chunk
    voff_b[i] = layout_b ? (o / kPerRt) * (32 * rowbytes) + (o % kPerRt / kPer) * 3072 + half * 1536 + (o % kPer) * 16 : r * rowbytes + p * 16;
  }
#pragma unroll
  for (int i = 0; i < NAL; i++) {
    const int o = i * 64 + lane, r = o / kPieces, p = swz(o - r * kPieces, r);
    voff_a[i] = r * rowbytes + p * 16;
  }
  // scale loads: lane l fetches the 16 bytes (four K-tiles) of row l % 32 (both halves of the wave fetch the same rows;
  // 64 or more rows of A: of row l, l + 64; 64 rows of B: of row l)
  const int ra = AR == 16 ? (r32 & 15) : r32;  // AR = 16: lanes 16-31 mirror rows 0-15 (their outputs are never stored)
  const int rb = BR == 16 ? (r32 & 15) : r32;  // BR = 16: likewise for B
  const int voff_bs = BR == 64 ? (layout_b ? h * (nk4 * 512) + r32 * 16 : lane * sbytes) : layout_b ? (half * 16 + rb) * 16 : rb * sbytes;
  const int voff_as = (AR >= 64 ? lane : r32) * sbytes;

  const uint32_t buf = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem + wave * kBuf;
  const uint8_t* bufp = smem + wave * kBuf;
  // LDS read offsets of this lane: K-tile u, piece c of its half (pieces 3h .. 3h+2 of the K-tile)
  int b_rd[KT][3], a_rd[KT][3];
#pragma unroll
  for (int u = 0; u < KT; u++)
#pragma unroll
    for (int c = 0; c < 3; c++) {
      const int p = u * 6 + 3 * h + c;
      b_rd[u][c] = layout_b ? u * ((BR == 16 ? 16 : 32) * 96) + rb * 96 + ((3 * h + c) ^ ((rb >> 3) & 1)) * 16 : rb * kRow + swz(p, rb) * 16;
      a_rd[u][c] = kAOff + ra * kRow + swz(p, ra) * 16;
    }

  // chunks of this workgroup: [c0, c1); of this wave: c0 + wave, c0 + wave + NW, ...
  const int nchunks = nkt / KT, cps = (nchunks + nsplit - 1) / nsplit;
  const int c0 = split * cps, c1 = min(nchunks, c0 + cps);
  const int mine = c0 + wave < c1 ? (c1 - c0 - wave + NW - 1) / NW : 0;

  // B's part of a chunk (NBL + 1 loads) into B buffer `par`, and A's part (NAL + NAS loads)
  auto issue_b = [&](int chunk, int par) __attribute__((always_inline)) {
    const int sg = KT == 4 ? chunk : chunk >> 1;  // the scales come in groups of four K-tiles
    const int sosb = __builtin_amdgcn_readfirstlane(layout_b ? sg * 512 : sg * 16);
    const uint32_t pb = __builtin_amdgcn_readfirstlane(par);
    dma16(rBs, buf + kScOff + pb * 1024, voff_bs, sosb);
    const int sob = __builtin_amdgcn_readfirstlane(layout_b ? chunk * (KT * 3072) : chunk * kRow);
#pragma unroll
    for (int i = 0; i < NBL; i++) dma16(rB, buf + pb * kBBuf + i * 1024, voff_b[i], sob);
  };
  auto issue_a = [&](int chunk) __attribute__((always_inline)) {
    const int sg = KT == 4 ? chunk : chunk >> 1;
    const int sos = __builtin_amdgcn_readfirstlane(sg * 16);
#pragma unroll
    for (int i = 0; i < NAS; i++) dma16(rAs, buf + kAScOff + i * 1024, voff_as + i * 64 * sbytes, sos);
    const int so = __builtin_amdgcn_readfirstlane(chunk * kRow);
#pragma unroll
    for (int i = 0; i < NAL; i++) dma16(rA, buf + kAOff + i * 1024, voff_a[i], so);
  };

  v16f acc[TT];
#pragma unroll
  for (int t = 0; t < TT; t++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[t][e] = 0.f;

  if (mine > 0) {
    // queue order: B(0), A(0), B(1), A(1), B(2), ...: with DB = 2 chunk j is read once everything up to A(j) has landed,
    // while B(j+1), the youngest batch, stays in flight
    issue_b(c0 + wave, 0);
    issue_a(c0 + wave);
    if (DB == 2 && mine > 1) issue_b(c0 + wave + NW, 1);
    for (int j = 0; j < mine; j++) {
      if (DB == 2 && j + 1 < mine) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NBL + 1) : "memory");
      else wait_vmcnt<0>();
      const int par = DB == 2 ? j & 1 : 0;
      const uint8_t* bufb = bufp + par * kBBuf;
      v4i sc_b[TB], sc_a[TA];
      v4i fb[TB][KT][3], fa[TA][KT][3];
#pragma unroll
      for (int tb = 0; tb < TB; tb++) sc_b[tb] = *reinterpret_cast<const v4i*>(bufp + kScOff + par * 1024 + (tb * 32 + rb) * 16);
      const bool odd = KT == 2 && ((c0 + wave + j * NW) & 1);  // half chunks: which two of the four scale bytes
#pragma unroll
      for (int t = 0; t < TA; t++) sc_a[t] = *reinterpret_cast<const v4i*>(bufp + kAScOff + (t * 32 + ra) * 16);
#pragma unroll
      for (int u = 0; u < KT; u++)
#pragma unroll
        for (int c = 0; c < 3; c++) {
#pragma unroll
          for (int tb = 0; tb < TB; tb++) fb[tb][u][c] = *reinterpret_cast<const v4i*>(bufb + b_rd[u][c] + tb * (kBBuf / 2));
#pragma unroll
          for (int t = 0; t < TA; t++) fa[t][u][c] = *reinterpret_cast<const v4i*>(bufp + a_rd[u][c] + t * (32 * kRow));
        }
      // the buffer is about to be refilled: its reads must have left LDS
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      if (DB == 2) {
        if (j + 1 < mine) issue_a(c0 + wave + (j + 1) * NW);
        if (j + 2 < mine) issue_b(c0 + wave + (j + 2) * NW, par);
      } else if (j + 1 < mine) {
        issue_b(c0 + wave + (j + 1) * NW, 0);
        issue_a(c0 + wave + (j + 1) * NW);
      }
#pragma unroll
      for (int u = 0; u < KT; u++)
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
          const int sb = (uint32_t)(KT == 4 ? sc_b[tb][u] : odd ? sc_b[tb][u + 2] : sc_b[tb][u]) >> (16 * h);
          const v8i b0 = __builtin_shufflevector(fb[tb][u][0], fb[tb][u][1], 0, 1, 2, 3, 4, 5, -1, -1);
          const v8i b1 = __builtin_shufflevector(fb[tb][u][1], fb[tb][u][2], 2, 3, 4, 5, 6, 7, -1, -1);
#pragma unroll
          for (int t = 0; t < TA; t++) {
            const int sa = (uint32_t)(KT == 4 ? sc_a[t][u] : odd ? sc_a[t][u + 2] : sc_a[t][u]) >> (16 * h);
            const v8i a0 = __builtin_shufflevector(fa[t][u][0], fa[t][u][1], 0, 1, 2, 3, 4, 5, -1, -1);
            const v8i a1 = __builtin_shufflevector(fa[t][u][1], fa[t][u][2], 2, 3, 4, 5, 6, 7, -1, -1);
            acc[t * TB + tb] = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc[t * TB + tb], sb, sa);
            acc[t * TB + tb] = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc[t * TB + tb], sb, sa);
          }
        }
    }
  }

  // sum the K-slices: register e of lane l is C[m = 32 t + l % 32][n = 32 tb + 8*(e/4) + 4*(l/32) + e%4] of accumulator tile t * TB + tb.
  // The buffers double as the reduction buffer once every wave has drained its loads.
  __syncthreads();
  float* part = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int t = 0; t < TT; t++)
#pragma unroll
    for (int e = 0; e < 16; e++) part[((wave * TT + t) * 16 + e) * 64 + lane] = acc[t][e];
  __syncthreads();
  const bool has_ep = epilogue_any(ep);
  if (nsplit > 1) {
    // K split between workgroups: every workgroup leaves its partial tile in the workspace; the one that arrives last
    // (a counter per tile) adds them up in split order, so the result does not depend on who that is.  The other
    // workgroups may run on XCDs with L2s of their own: partial tiles and counter are written and read with
    // device-scope atomic accesses, which go past those caches, instead of device-scope fences, which write back and
    // invalidate a whole L2 per wave (measured: 0.2 us per workgroup, one after the other).
    // (a workgroup's partial result is TT tiles of 4 KB: idx = (tile of the wave * 16 + register) * 64 + lane)
    float* mine_ws = ws_part + ((size_t)tile * nsplit + split) * (TT * 1024);
    for (int idx = tid; idx < TT * 1024; idx += NW * 64) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < NW; w++) t += part[w * (TT * 1024) + idx];
      __hip_atomic_store(mine_ws + idx, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    wait_vmcnt<0>();  // stores count there too: the partial tile has arrived before the counter moves
    __syncthreads();
    int* flag = reinterpret_cast<int*>(smem + NW * TT * 16 * 64 * 4);  // behind the partial tiles
    if (tid == 0) *flag = __hip_atomic_fetch_add(ws_cnt + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nsplit - 1;
    __syncthreads();
    if (!*flag) return;
    const float* all = ws_part + (size_t)tile * nsplit * (TT * 1024);
    for (int idx = tid; idx < TT * 1024; idx += NW * 64) {
      const int tt = idx >> 10, e = (idx >> 6) & 15, l = idx & 63;
      float t = 0.f;
      for (int q = 0; q < nsplit; q++) t += __hip_atomic_load(all + q * (TT * 1024) + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int m = (tt / TB) * 32 + (l & 31);
      const int nl = (tt % TB) * 32 + 8 * (e >> 2) + 4 * (l >> 5) + (e & 3);
      const long nn = (long)n0 + nl;
      if (m < M && nl < BR && nn < N) store1(C + (long)m * N + nn, has_ep ? epilogue_apply(ep, t, m, nn) : t);
    }
    if (tid == 0) __hip_atomic_store(ws_cnt + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    return;
  }
  for (int idx = tid; idx < TT * 1024; idx += NW * 64) {
    const int tt = idx >> 10, e = (idx >> 6) & 15, l = idx & 63;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) s += part[w * (TT * 1024) + idx];
    const int m = (tt / TB) * 32 + (l & 31);
    const int nl = (tt % TB) * 32 + 8 * (e >> 2) + 4 * (l >> 5) + (e & 3);
    const long nn = (long)n0 + nl;
    if (m < M && nl < BR && nn < N) store1(C + (long)m * N + nn, has_ep ? epilogue_apply(ep, s, m, nn) : s);
  }
}

bool gemm_skinny_supports(const GemmArgs& g) {
  // K % 512: chunks of four K-tiles are whole (three 128-byte lines per row, 16 scale bytes per row)
  return g.layout_a == 0 && g.M >= 1 && g.M <= 128 && g.N >= 1 && g.K >= 512 && g.K % 512 == 0 && (long)128 * (g.K / 4 * 3) < (1L << 31) && operands_aligned16(g);
}

// Workspace of the K split: 4 KB of partial tile per (tile, split) and a counter per tile that is zero between
// launches.  One per (device, stream), taken from the stream-ordered allocator on the caller's stream at the first split
// launch there (no device-wide synchronisation) and kept until release_split_workspaces(): launches on one stream are
// ordered, so they can share it; launches on different streams get different ones.  (Two graphs captured on one stream
// and replayed at the same time on different streams would share theirs: replay them on one stream, or switch the split
// off with geometry 7 - 9.)  No allocation is possible while the stream is being captured: a capture without a workspace
// runs unsplit.  At most kWsMax workspaces exist at a time; a further stream runs unsplit.
namespace {
constexpr int kWsSlots = 512, kWsTiles = 512;  // partial tiles of 4 KB and tiles of C a workspace holds (the automatic choice never needs more)
constexpr size_t kWsMax = 64;
struct SplitWs {
  float* part = nullptr;
  int* cnt = nullptr;
  bool pinned = false;  // handed out while its stream was being captured: a graph holds the pointers, the block is never freed
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, SplitWs> g_ws;

__global__ void clear_counters_kernel(int* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

SplitWs split_workspace(hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return {};
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  const bool capturing = hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone;
  if (capturing) (void)hipGetLastError();
  auto it = g_ws.find({dev, s});
  if (it != g_ws.end()) {
    if (capturing) it->second.pinned = true;
    return it->second;
  }
  if (g_ws.size() >= kWsMax || capturing) return {};
  SplitWs w;
  uint8_t* base = nullptr;
  if (hipMallocAsync((void**)&base, (size_t)kWsSlots * 4096 + kWsTiles * sizeof(int), s) != hipSuccess || !base) {
    (void)hipGetLastError();
    return {};
  }
  w.part = reinterpret_cast<float*>(base);
  w.cnt = reinterpret_cast<int*>(base + (size_t)kWsSlots * 4096);
  // cleared on the caller's stream: ordered before the launch that follows
  clear_counters_kernel<<<(kWsTiles + 255) / 256, 256, 0, s>>>(w.cnt, kWsTiles);
  if (hipGetLastError() != hipSuccess) {
    (void)hipFreeAsync(base, s);
    return {};
  }
  g_ws[{dev, s}] = w;
  return w;
}

// The scratch memory of the entry point that allocates nothing (launch_gemm_skinny with GemmArgs::no_alloc): partial
// tiles and counters of the K split live in the array `scratch` at the top of this file, of which every GPU holds its
// own copy at its own address.  The address is looked up once per device, with that device current, and only that
// pointer is handed to kernels.
unsigned char* g_scratch_ptr[64] = {};
hipError_t scratch_of_current_device(unsigned char** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}
}  // namespace

hipError_t release_split_workspaces() {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  if (g_ws.empty()) return hipSuccess;
  int cur = 0;
  (void)hipGetDevice(&cur);
  hipError_t first = hipSuccess;
  for (auto& kv : g_ws) {
    if (kv.second.pinned) continue;  // recorded in a graph: stays allocated until the process ends
    // stream-ordered: the memory goes back once the work queued on that stream so far has finished with it
    (void)hipSetDevice(kv.first.first);
    const hipError_t e = hipFreeAsync(kv.second.part, kv.first.second);
    if (e != hipSuccess && first == hipSuccess) first = e;
  }
  g_ws.clear();
  (void)hipSetDevice(cur);
  return first;
}

// Geometry.  Few rows of B (N / 32 workgroups would leave CUs idle): a workgroup takes 16 rows of B, and the K range
// is split between 2, 4 or 8 workgroups while that still fits the CUs and leaves every wave kMinChunks chunks.  More
// than one workgroup per CU (N / 32 above the CU count): half as many waves per workgroup, so that two workgroups share
// a CU and one's first loads run under the other's stream (a workgroup with a short K range is mostly load latency);
// with at most 16 chunks of K and up to 16 rows of A, two waves per workgroup (eight workgroups share a CU, each wave
// streams a longer part of K: measured 5 - 13 % at N = 14336 .. 28672, K = 4096 .. 8192, nothing beyond N = 32768).
// 64 rows of B per workgroup (17 - 128 rows of A): every fragment of A meets two tiles of B, so a workgroup pulls half
// the bytes of A from L2 per byte of B; the K range is split in two (or four) where N / 64 alone would leave CUs idle.
// skinny_geometry: 1 - 3 fix the workgroup shape without a split; 4 + 3 * b + log2(split) - 1 (b = 0: 32 rows of B,
// b = 1: 16 rows) fixes both; 10 = two waves per workgroup; 11 - 13 = 64 rows of B with K unsplit / split in 2 / in 4.
struct SkinnyPlan {
  int geo, want;   // workgroup shape (1: 32 rows of B, 2: 16 rows, 3: half the waves, 5: two waves, 6: 64 rows of B) and wanted K split
  unsigned tiles;  // tiles of C (one arrival counter each when K is split)
  unsigned slots;  // 4 KB partial tiles the split leaves in the workspace
};
static SkinnyPlan skinny_plan(const GemmArgs& g) {
  const unsigned wgs32 = (g.N + 31) / 32;
  const int nchunks = g.K / 512, nw = g.M <= 16 ? 8 : 6;
  int geo, want = 1;
  if (g.skinny_geometry >= 11 && g.skinny_geometry <= 13) {
    geo = 6, want = 1 << (g.skinny_geometry - 11);
  } else if (g.skinny_geometry == 0 && !g.force_split && g.M > 16 && g.M <= 64 && (g.N + 63) / 64 >= 256 && g.K >= 8192) {
    // wide N, long K, 17 - 64 rows of A: 64 rows of B per workgroup (measured 5 - 13 % at N = 16384 .. 57344, K >= 8192;
    // 3 - 9 % slower at K = 4096, where a workgroup's K range is too short for its fewer, larger chunks)
    geo = 6;
  } else if (g.M > 32) {
    // 33 - 128 rows of A: two or four accumulator tiles per wave, four waves or two (two workgroups per CU), no K split
    geo = g.skinny_geometry == 3 || (g.skinny_geometry == 0 && wgs32 > 256) ? 3 : 1;
  } else if (g.skinny_geometry == 10) {
    geo = g.M <= 16 ? 5 : 3;  // two waves per workgroup (up to 16 rows of A)
  } else if (g.skinny_geometry >= 4) {
    geo = 1 + (g.skinny_geometry - 4) / 3;
    want = 2 << ((g.skinny_geometry - 4) % 3);
  } else if (g.skinny_geometry) {
    geo = g.skinny_geometry;
  } else if (g.force_split) {
    // the caller fixes the split (1, 2, 4 or 8); the workgroup shape follows N as in the automatic choice for split shapes
    geo = wgs32 <= 128 ? 2 : 1;
    want = g.force_split;
  } else {
    geo = wgs32 <= 128 ? 2 : wgs32 <= 256 ? 1 : g.M <= 16 && wgs32 <= 1024 && nchunks <= 16 ? 5 : 3;
    constexpr int kMinChunks = 3;  // measured: below this the 2.5 us of the second phase outweigh the wider stream
    const unsigned tiles = geo == 2 ? (g.N + 15) / 16 : wgs32;
    if (geo != 3)
      while (want < 8 && tiles * want * 2 <= 256 && nchunks / (want * 2) >= kMinChunks * nw) want *= 2;
  }
  const unsigned tiles = geo == 2 ? (unsigned)(g.N + 15) / 16 : geo == 6 ? (unsigned)(g.N + 63) / 64 : wgs32;
  const unsigned tt = geo == 6 ? 2 * (g.M > 64 ? 4 : g.M > 32 ? 2 : 1) : 1;  // accumulator tiles per workgroup
  return {geo, want, tiles, tiles * want * tt};
}

// Does the K split this call would use fit the scratch array of the entry point that allocates nothing?
bool gemm_skinny_scratch_fits(const GemmArgs& g) {
  const SkinnyPlan p = skinny_plan(g);
  return p.want <= 1 || (p.tiles <= (unsigned)kScratchTiles && p.slots <= (unsigned)kScratchSlots);
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  typedef typename Out::type T;
  const SkinnyPlan plan = skinny_plan(g);
  const int geo = plan.geo, want = plan.want;
  int nsplit = 1;
  SplitWs ws;
  const unsigned tiles = plan.tiles;
  if (g.no_alloc) {
    // nothing is allocated: the split uses this device's scratch array, whose counters are cleared by a small kernel in
    // front of the launch (the array keeps whatever the previous call left)
    if (want > 1) {
      if (tiles > (unsigned)kScratchTiles || plan.slots > (unsigned)kScratchSlots) return hipErrorInvalidValue;  // the entry point checked this already
      unsigned char* base = nullptr;
      const hipError_t e = scratch_of_current_device(&base);
      if (e != hipSuccess) return e;
      ws.part = reinterpret_cast<float*>(base);
      ws.cnt = reinterpret_cast<int*>(base + (size_t)kScratchSlots * 4096);
      clear_counters_kernel<<<(tiles + 255) / 256, 256, 0, s>>>(ws.cnt, (int)tiles);
      const hipError_t ce = hipGetLastError();
      if (ce != hipSuccess) return ce;
      nsplit = want;
    }
  } else if (want > 1 && tiles <= (unsigned)kWsTiles && plan.slots <= (unsigned)kWsSlots) {
    ws = split_workspace(s);
    if (ws.part) nsplit = want;
  }
#define MXFP6_SK(AR, NW, BR) MXFP6_SKD(AR, NW, BR, 1)
#define MXFP6_SKD(AR, NW, BR, DB) \
  gemm_skinny_kernel<FA, FB, Out, AR, NW, BR, DB><<<(g.N + BR - 1) / BR * nsplit, NW * 64, 0, s>>>( \
      g.A, g.B, g.As, g.Bs, (T*)g.C, g.M, g.N, g.K, g.layout_b, g.ep, nsplit, ws.part, ws.cnt)
  // two chunks of B per wave (17 - 32 and 65 - 128 rows of A: measured 3 - 15 % and 3 - 6 %); forced geometry 1: one
  const bool db = g.skinny_geometry != 1;
  if (geo == 6) {
    if (g.M > 64) MXFP6_SK(128, 4, 64); else if (g.M > 32) MXFP6_SK(64, 3, 64); else MXFP6_SK(32, 4, 64);
  } else if (g.M > 64) {
    if (geo == 3) MXFP6_SK(128, 2, 32); else if (db) MXFP6_SKD(128, 4, 32, 2); else MXFP6_SK(128, 4, 32);
  } else if (g.M > 32) {
    if (geo == 3) MXFP6_SK(64, 2, 32); else MXFP6_SK(64, 4, 32);  // two chunks of B and three waves: measured level with this
  } else if (g.M <= 16) {
    if (geo == 2) MXFP6_SK(16, 8, 16); else if (geo == 3) MXFP6_SK(16, 4, 32); else if (geo == 5) MXFP6_SK(16, 2, 32); else MXFP6_SK(16, 8, 32);
  } else {
    if (geo == 2) MXFP6_SK(32, 6, 16); else if (geo == 3) MXFP6_SK(32, 3, 32); else if (db && geo == 1) MXFP6_SKD(32, 4, 32, 2); else MXFP6_SK(32, 6, 32);
  }
#undef MXFP6_SKD
#undef MXFP6_SK
  return hipGetLastError();
}

hipError_t launch_gemm_skinny(const GemmArgs& g, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (g.fmt_a == FA && g.fmt_b == FB) return g.f32out ? launch<FA, FB, OutF32>(g, s) : launch<FA, FB, OutBf16>(g, s);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipErrorInvalidValue;
}

}  // namespace mxfp6
