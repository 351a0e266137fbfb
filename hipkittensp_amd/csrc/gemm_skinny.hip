// Skinny-M (decode-shaped) MXFP6 GEMM for gfx950: M <= 32, HBM-bound.
//
// Every byte of B (weights) and of its scales is read exactly once, straight from global memory
// into the MFMA source registers (16-byte loads of the packed rows; no unpacking, no LDS staging:
// with M <= 32 a B element meets the tensor core once).  A (the few activation rows) is re-read
// from L2 by every wave.  One workgroup owns 32 consecutive rows of B (32 output columns) and
// splits K over its 8 waves; the 8 partial 32x32 tiles are summed through LDS, so no global
// scratch and no atomics are needed.  Each wave keeps four K-tiles (4 x 48 bytes per lane per
// operand) in flight, about 100 KB per CU, which is what HBM latency x bandwidth asks for.
//
// The reference has no kernel for this shape (its GEMMs need M, N multiples of the 256 tile,
// analysis/bf16_gemm/mi325x/kernel_8192.cpp:24-32); the MFMA operand conventions are those of the
// tiled kernel.  Algorithmic bytes per launch: 0.75*K*(M+N) + (K/32)*(M+N) + 2*M*N.
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

constexpr int kSkinnyWaves = 8;
constexpr int kPF = 4;  // K-tiles in flight per wave

struct Frag {
  v4i b[3], a[3];  // the lane's 48 bytes (two 32-element K-blocks) of its B row and A row
  int sb, sa;      // the two E8M0 bytes of those K-blocks, B and A
};

// Loads are issued from inline assembly and waited for by hand: the compiler's own counter
// placement drains the whole queue once per loop iteration, which leaves HBM idle while the
// MFMAs run.  The wait takes the stage's registers as read-write operands so that no use can be
// scheduled above it.
__device__ __forceinline__ v4i load128_stream(const __amdgpu_buffer_rsrc_t& r, uint32_t voff, int soff) {
  v4i d;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen nt" : "=v"(d) : "v"(voff), "s"(r), "s"(soff) : "memory");
  return d;
}
__device__ __forceinline__ v4i load128(const __amdgpu_buffer_rsrc_t& r, uint32_t voff, int soff) {
  v4i d;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(d) : "v"(voff), "s"(r), "s"(soff) : "memory");
  return d;
}
__device__ __forceinline__ int load16(const __amdgpu_buffer_rsrc_t& r, uint32_t voff, int soff) {
  int d;
  asm volatile("buffer_load_ushort %0, %1, %2, %3 offen" : "=v"(d) : "v"(voff), "s"(r), "s"(soff) : "memory");
  return d;
}
constexpr int kLoadsPerStage = 8;
template <int N>
__device__ __forceinline__ void wait_stage(Frag& f) {
  asm volatile("s_waitcnt vmcnt(%8)"
               : "+v"(f.b[0]), "+v"(f.b[1]), "+v"(f.b[2]), "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.sb), "+v"(f.sa)
               : "n"(N)
               : "memory");
}

template <int FA, int FB, typename Out>
__global__ __launch_bounds__(kSkinnyWaves * 64) void gemm_skinny_kernel(const uint8_t* __restrict__ A,
                                                                        const uint8_t* __restrict__ B,
                                                                        const uint8_t* __restrict__ As,
                                                                        const uint8_t* __restrict__ Bs,
                                                                        typename Out::type* __restrict__ C, int M, int N, int K) {
  __shared__ float part[kSkinnyWaves][16][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int nkt = K / 128, sbytes = K / 32, rowbytes = K / 4 * 3;
  const long n = (long)blockIdx.x * 32 + r32;
  // K-tiles [t0, t1) of this wave
  const int per = (nkt + kSkinnyWaves - 1) / kSkinnyWaves;
  const int t0 = min(wave * per, nkt), t1 = min(t0 + per, nkt);

  // buffer resources bound the operands: a lane whose row does not exist (n >= N, m >= M) points
  // past the end and reads zeros -- no divergent control flow around the loads
  const __amdgpu_buffer_rsrc_t rB = make_rsrc(B, (uint32_t)N * (uint32_t)rowbytes);
  const __amdgpu_buffer_rsrc_t rA = make_rsrc(A, (uint32_t)M * (uint32_t)rowbytes);
  const __amdgpu_buffer_rsrc_t rBs = make_rsrc(Bs, (uint32_t)N * (uint32_t)sbytes);
  const __amdgpu_buffer_rsrc_t rAs = make_rsrc(As, (uint32_t)M * (uint32_t)sbytes);
  const uint32_t kOob = 0xFFFFFF00u;
  const uint32_t vb = n < N ? (uint32_t)n * rowbytes + 48 * h : kOob;
  const uint32_t va = r32 < M ? (uint32_t)r32 * rowbytes + 48 * h : kOob;
  const uint32_t vbs = n < N ? (uint32_t)n * sbytes + 2 * h : kOob;
  const uint32_t vas = r32 < M ? (uint32_t)r32 * sbytes + 2 * h : kOob;

  auto load = [&](Frag& f, int t) {
    const int so = __builtin_amdgcn_readfirstlane(t * 96), ss = __builtin_amdgcn_readfirstlane(t * 4);
    // B is streamed once: non-temporal; A is shared by every wave: default policy
#pragma unroll
    for (int c = 0; c < 3; c++) {
      f.b[c] = load128_stream(rB, vb, so + 16 * c);
      f.a[c] = load128(rA, va, so + 16 * c);
    }
    f.sb = load16(rBs, vbs, ss);
    f.sa = load16(rAs, vas, ss);
  };

  v16f acc;
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.f;

  Frag f[kPF];
  auto use = [&](Frag& g) {
    const v8i b0 = __builtin_shufflevector(g.b[0], g.b[1], 0, 1, 2, 3, 4, 5, -1, -1);
    const v8i b1 = __builtin_shufflevector(g.b[1], g.b[2], 2, 3, 4, 5, 6, 7, -1, -1);
    const v8i a0 = __builtin_shufflevector(g.a[0], g.a[1], 0, 1, 2, 3, 4, 5, -1, -1);
    const v8i a1 = __builtin_shufflevector(g.a[1], g.a[2], 2, 3, 4, 5, 6, 7, -1, -1);
    acc = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc, g.sb, g.sa);
    acc = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc, g.sb, g.sa);
  };
  const int nt = t1 - t0;
  int t = 0;
  if (nt >= 2 * kPF) {
    // prologue, then a steady state in which every stage is consumed and at once refilled with
    // the tile kPF ahead: kPF-1 stages (3 x 8 loads) are always in flight
#pragma unroll
    for (int s = 0; s < kPF; s++) load(f[s], t0 + s);
    for (; t + 2 * kPF <= nt; t += kPF) {
#pragma unroll
      for (int s = 0; s < kPF; s++) {
        wait_stage<(kPF - 1) * kLoadsPerStage>(f[s]);
        use(f[s]);
        load(f[s], t0 + t + kPF + s);
      }
    }
    // drain the kPF stages still in flight
    wait_stage<3 * kLoadsPerStage>(f[0]); use(f[0]);
    wait_stage<2 * kLoadsPerStage>(f[1]); use(f[1]);
    wait_stage<1 * kLoadsPerStage>(f[2]); use(f[2]);
    wait_stage<0>(f[3]); use(f[3]);
    static_assert(kPF == 4, "drain sequence is written for four stages");
    t += kPF;
  }
  // remainder (and short K): one tile at a time
  for (; t < nt; t++) {
    load(f[0], t0 + t);
    wait_stage<0>(f[0]);
    use(f[0]);
  }

  // sum the K-slices: register e of lane l is C[m = l % 32][n = 8*(e/4) + 4*(l/32) + e%4]
#pragma unroll
  for (int e = 0; e < 16; e++) part[wave][e][lane] = acc[e];
  __syncthreads();
  // 512 threads, 1024 outputs: thread handles registers e and e + 8 of its lane
#pragma unroll
  for (int half = 0; half < 2; half++) {
    const int e = (tid >> 6) + 8 * half;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kSkinnyWaves; w++) s += part[w][e][lane];
    const int m = lane & 31;
    const long nn = (long)blockIdx.x * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
    if (m < M && nn < N) store1(C + (long)m * N + nn, s);
  }
}

bool gemm_skinny_supports(const GemmArgs& g) {
  return g.M >= 1 && g.M <= 32 && g.N >= 1 && g.K >= 128 && g.K % 128 == 0 && (long)g.N * (g.K / 4 * 3) < 0xFFFFFF00L;
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  gemm_skinny_kernel<FA, FB, Out><<<(g.N + 31) / 32, kSkinnyWaves * 64, 0, s>>>(g.A, g.B, g.As, g.Bs, (typename Out::type*)g.C, g.M, g.N, g.K);
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
