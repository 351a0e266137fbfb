// Skinny-M (decode-shaped) MXFP6 GEMM for gfx950: M <= 32, bound by HBM.
//
// Every byte of B (weights) is read from HBM once.  One workgroup owns 32 consecutive rows of B
// (32 output columns) and splits K over its waves in chunks of four K-tiles (4 x 128 elements =
// 384 bytes per row = three whole 128-byte lines), dealt round-robin: wave w takes chunks w, w+NW, ...
// so the workgroup streams one contiguous K range of its 32 rows and no cache line is shared
// between chunks.  With a tile-major B the 32 rows x K of a workgroup are one contiguous run of HBM.  Each wave owns a private 4-stage LDS ring (one stage per K-tile of a chunk):
//   global --buffer_load_dwordx4 ... lds--> LDS --ds_read_b128--> MFMA sources
// with the same lane->address map as the tiled kernel (consecutive lanes fetch consecutive 16-byte
// pieces of a row; row-major 96-byte LDS rows with a pair swap that makes the reads conflict-free).
// Staging through LDS is what lets the loads be coalesced: the MFMA wants lane = row, the memory
// system wants lane = consecutive bytes.  A's rows (M <= 32) are staged the same way from L2.  The
// E8M0 bytes of a chunk are 16 bytes per row: one 16-byte load per lane per chunk, kept in VGPRs.
// All loads are issued from inline assembly and waited for with hand-counted vmcnt, four K-tiles
// ahead.  The partial 32x32 tiles of the waves are summed through LDS: no scratch, no atomics.
//
// The reference has no kernel for this shape (its GEMMs need M, N multiples of the 256 tile,
// analysis/bf16_gemm/mi325x/kernel_8192.cpp:24-32).  Algorithmic bytes per launch:
// 0.75*K*(M+N) + (K/32)*(M+N) + 2*M*N.
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

namespace {

constexpr int kStagesSk = 4;  // = K-tiles per chunk

__device__ __forceinline__ void dma16_sk(const __amdgpu_buffer_rsrc_t& rsrc, uint32_t lds_base, int voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}
__device__ __forceinline__ v4i load128_sk(const __amdgpu_buffer_rsrc_t& r, int voff, int soff) {
  v4i d;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(d) : "v"(voff), "s"(r), "s"(soff) : "memory");
  return d;
}
// wait until at most N of this wave's loads are outstanding; the scale registers ride along as
// read-write operands so that no use of them can be scheduled above the wait
template <int N>
__device__ __forceinline__ void wait_loads(v4i& s0, v4i& s1) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(s0), "+v"(s1) : "n"(N) : "memory");
}

}  // namespace

// AR = rows of A staged per K-tile (16 or 32); NW = waves per workgroup
template <int FA, int FB, typename Out, int AR, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                              const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bs,
                                                              typename Out::type* __restrict__ C, int M, int N, int K, int layout_b) {
  constexpr int kBTile = 32 * 96, kATile = AR * 96, kStage = kBTile + kATile, kRing = kStagesSk * kStage;
  constexpr int kADma = (kATile + 1023) / 1024;  // direct loads per A tile (the last one half full when AR = 16)
  constexpr int kDmaPerTile = 3 + kADma;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NW * kRing];
  static_assert(NW * kRing <= 163840 && NW * kRing >= NW * 16 * 64 * 4, "LDS budget (ring doubles as the reduction buffer)");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int nkt = K / 128, sbytes = K / 32, rowbytes = K / 4 * 3;
  const int n0 = blockIdx.x * 32;
  const int nrows = min(32, N - n0);

  // rows that do not exist (n >= N, m >= M) lie past the end of the resource and read as zeros
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(B + (size_t)n0 * rowbytes, (uint32_t)nrows * rowbytes);
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A, (uint32_t)M * rowbytes);
  // tile-major B: this workgroup's 32 rows are one row-tile, whose scales are nk4 chunks of 512 bytes (row r at r * 16)
  const int nk4 = (nkt + 3) / 4;
  const __amdgpu_buffer_rsrc_t rBs = layout_b ? make_rsrc(Bs + (size_t)blockIdx.x * nk4 * 512, (uint32_t)nk4 * 512)
                                              : make_rsrc(Bs + (size_t)n0 * sbytes, (uint32_t)nrows * sbytes);
  const __amdgpu_buffer_rsrc_t rAs = make_rsrc(As, (uint32_t)M * sbytes);

  // direct-load address map: LDS slot o (16 bytes) of a tile holds chunk (o%6) ^ ((row>>3)&1) of row o/6
  int voff[3];
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int o = i * 64 + lane, r = o / 6, c = (o - r * 6) ^ ((r >> 3) & 1);
    voff[i] = r * rowbytes + c * 16;
  }
  // tile-major B: the 32-row tile is stored in LDS image order, a load is one contiguous KiB
  int voff_bt[3];
#pragma unroll
  for (int i = 0; i < 3; i++) voff_bt[i] = layout_b ? (i * 64 + lane) * 16 : voff[i];
  const int voff_bs = layout_b ? r32 * 16 : r32 * sbytes, voff_as = (AR == 16 ? (r32 & 15) : r32) * sbytes;

  const uint32_t ring = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem + wave * kRing;
  const uint8_t* ringp = smem + wave * kRing;
  const int sw = (r32 >> 3) & 1;
  int b_rd[3], a_rd[3];
#pragma unroll
  for (int c = 0; c < 3; c++) {
    b_rd[c] = r32 * 96 + ((3 * h + c) ^ sw) * 16;
    const int ra = AR == 16 ? (r32 & 15) : r32;  // AR = 16: lanes 16-31 mirror rows 0-15 (their outputs are never stored)
    a_rd[c] = kBTile + ra * 96 + ((3 * h + c) ^ ((ra >> 3) & 1)) * 16;
  }

  // chunks of this wave: wave, wave + NW, ...
  const int nchunks = (nkt + 3) / 4;
  const int mine = wave < nchunks ? (nchunks - wave + NW - 1) / NW : 0;

  v4i sc_b_next, sc_a_next, sc_b, sc_a;
  sc_b_next = sc_a_next = sc_b = sc_a = v4i{0, 0, 0, 0};

  auto issue_scales = [&](int chunk) {  // 16 scale bytes per row: the chunk's four K-tiles
    const int so = __builtin_amdgcn_readfirstlane(chunk * 16);
    const int sob = __builtin_amdgcn_readfirstlane(layout_b ? chunk * 512 : chunk * 16);
    sc_b_next = load128_sk(rBs, voff_bs, sob);
    sc_a_next = load128_sk(rAs, voff_as, so);
  };
  auto issue_tile = [&](int chunk, int u) {  // K-tile u of a chunk into stage u
    const int t = min(chunk * 4 + u, nkt - 1);  // past-the-end tiles re-read the last one and are never multiplied
    const int so = __builtin_amdgcn_readfirstlane(t * 96);
    const int sob = __builtin_amdgcn_readfirstlane(layout_b ? t * 3072 : t * 96);
    const uint32_t dst = ring + u * kStage;
#pragma unroll
    for (int i = 0; i < 3; i++) dma16_sk(rB, dst + i * 1024, voff_bt[i], sob);
    dma16_sk(rA, dst + kBTile, voff[0], so);
    if constexpr (kADma == 2) {
      if (lane < 32) dma16_sk(rA, dst + kBTile + 1024, voff[1], so);
    } else {
      dma16_sk(rA, dst + kBTile + 1024, voff[1], so);
      dma16_sk(rA, dst + kBTile + 2048, voff[2], so);
    }
  };

  v16f acc;
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.f;

  auto consume = [&](int chunk, int u) {
    if (chunk * 4 + u >= nkt) return;
    const uint8_t* st = ringp + u * kStage;
    v4i fb[3], fa[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
      fb[c] = *reinterpret_cast<const v4i*>(st + b_rd[c]);
      fa[c] = *reinterpret_cast<const v4i*>(st + a_rd[c]);
    }
    const int sb = (uint32_t)sc_b[u] >> (16 * h), sa = (uint32_t)sc_a[u] >> (16 * h);
    const v8i b0 = __builtin_shufflevector(fb[0], fb[1], 0, 1, 2, 3, 4, 5, -1, -1);
    const v8i b1 = __builtin_shufflevector(fb[1], fb[2], 2, 3, 4, 5, 6, 7, -1, -1);
    const v8i a0 = __builtin_shufflevector(fa[0], fa[1], 0, 1, 2, 3, 4, 5, -1, -1);
    const v8i a1 = __builtin_shufflevector(fa[1], fa[2], 2, 3, 4, 5, 6, 7, -1, -1);
    acc = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc, sb, sa);
    acc = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc, sb, sa);
    // the stage is about to be refilled: its reads must have left LDS
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };

  if (mine > 0) {
    issue_scales(wave);
#pragma unroll
    for (int u = 0; u < 4; u++) issue_tile(wave, u);
    int j = 0;
    // steady state: waiting for tile (j,u) leaves the direct loads of the next three tiles in flight,
    // plus the two scale loads of chunk j+1 once they have been issued (u >= 1)
    for (; j + 1 < mine; j++) {
      const int chunk = wave + j * NW, next = chunk + NW;
      wait_loads<3 * kDmaPerTile>(sc_b_next, sc_a_next);
      sc_b = sc_b_next;
      sc_a = sc_a_next;
      consume(chunk, 0);
      issue_scales(next);
      issue_tile(next, 0);
#pragma unroll
      for (int u = 1; u < 4; u++) {
        wait_loads<3 * kDmaPerTile + 2>(sc_b_next, sc_a_next);
        consume(chunk, u);
        issue_tile(next, u);
      }
    }
    // last chunk: nothing more to issue
    const int chunk = wave + j * NW;
    wait_loads<3 * kDmaPerTile>(sc_b_next, sc_a_next);
    sc_b = sc_b_next;
    sc_a = sc_a_next;
    consume(chunk, 0);
    wait_loads<2 * kDmaPerTile>(sc_b_next, sc_a_next);
    consume(chunk, 1);
    wait_loads<1 * kDmaPerTile>(sc_b_next, sc_a_next);
    consume(chunk, 2);
    wait_loads<0>(sc_b_next, sc_a_next);
    consume(chunk, 3);
  }

  // sum the K-slices: register e of lane l is C[m = l % 32][n = 8*(e/4) + 4*(l/32) + e%4].
  // The ring doubles as the reduction buffer once every wave has drained its loads.
  __syncthreads();
  float* part = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int e = 0; e < 16; e++) part[(wave * 16 + e) * 64 + lane] = acc[e];
  __syncthreads();
  for (int idx = tid; idx < 1024; idx += NW * 64) {
    const int e = idx >> 6, l = idx & 63;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) s += part[(w * 16 + e) * 64 + l];
    const int m = l & 31;
    const long nn = (long)n0 + 8 * (e >> 2) + 4 * (l >> 5) + (e & 3);
    if (m < M && nn < N) store1(C + (long)m * N + nn, s);
  }
}

bool gemm_skinny_supports(const GemmArgs& g) {
  // K % 512: chunks of four K-tiles are whole (three 128-byte lines per row, 16 scale bytes per row)
  return g.layout_a == 0 && g.M >= 1 && g.M <= 32 && g.N >= 1 && g.K >= 512 && g.K % 512 == 0 && (long)32 * (g.K / 4 * 3) < (1L << 31);
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  const unsigned grid = (g.N + 31) / 32;
  if (g.M <= 16)
    gemm_skinny_kernel<FA, FB, Out, 16, 8><<<grid, 8 * 64, 0, s>>>(g.A, g.B, g.As, g.Bs, (typename Out::type*)g.C, g.M, g.N, g.K, g.layout_b);
  else
    gemm_skinny_kernel<FA, FB, Out, 32, 6><<<grid, 6 * 64, 0, s>>>(g.A, g.B, g.As, g.Bs, (typename Out::type*)g.C, g.M, g.N, g.K, g.layout_b);
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
