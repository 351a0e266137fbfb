// Skinny-M (decode-shaped) MXFP6 GEMM for gfx950: M <= 32, HBM-bound.
//
// Every byte of B (weights) and of its scales is read exactly once, straight from global memory
// into the MFMA source registers (16-byte loads of the packed rows; no unpacking, no LDS staging:
// with M <= 32 a B element meets the tensor core once).  A (the few activation rows) is re-read
// from L2 by every wave.  One workgroup owns 32 consecutive rows of B (32 output columns) and
// splits K over its 16 waves; the 16 partial 32x32 tiles are summed through LDS, so no global
// scratch and no atomics are needed.  Each wave keeps three K-tiles (3 x 48 bytes per lane per
// operand) in flight, about 100 KB per CU, which is what HBM latency x bandwidth asks for.
//
// The reference has no kernel for this shape (its GEMMs need M, N multiples of the 256 tile,
// analysis/bf16_gemm/mi325x/kernel_8192.cpp:24-32); the MFMA operand conventions are those of the
// tiled kernel.  Algorithmic bytes per launch: 0.75*K*(M+N) + (K/32)*(M+N) + 2*M*N.
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

constexpr int kSkinnyWaves = 16;
constexpr int kPF = 3;  // K-tiles in flight per wave

struct Frag {
  v4i b[3], a[3];  // the lane's 48 bytes (two 32-element K-blocks) of its B row and A row
};

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

  auto load = [&](Frag& f, int& sb, int& sa, int t) {
#pragma unroll
    for (int c = 0; c < 3; c++) {
      // B is streamed once: non-temporal; A is shared by every wave: default policy
      f.b[c] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rB, vb, t * 96 + 16 * c, 2));
      f.a[c] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rA, va, t * 96 + 16 * c, 0));
    }
    sb = __builtin_amdgcn_raw_buffer_load_b16(rBs, vbs, t * 4, 0);
    sa = __builtin_amdgcn_raw_buffer_load_b16(rAs, vas, t * 4, 0);
  };

  v16f acc;
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.f;

  Frag f[kPF];
  int sb[kPF], sa[kPF];
#pragma unroll
  for (int s = 0; s < kPF; s++)
    if (t0 + s < t1) load(f[s], sb[s], sa[s], t0 + s);

  for (int t = t0; t < t1; t += kPF) {
#pragma unroll
    for (int s = 0; s < kPF; s++) {
      if (t + s < t1) {
        const v8i b0 = __builtin_shufflevector(f[s].b[0], f[s].b[1], 0, 1, 2, 3, 4, 5, -1, -1);
        const v8i b1 = __builtin_shufflevector(f[s].b[1], f[s].b[2], 2, 3, 4, 5, 6, 7, -1, -1);
        const v8i a0 = __builtin_shufflevector(f[s].a[0], f[s].a[1], 0, 1, 2, 3, 4, 5, -1, -1);
        const v8i a1 = __builtin_shufflevector(f[s].a[1], f[s].a[2], 2, 3, 4, 5, 6, 7, -1, -1);
        const int csb = sb[s], csa = sa[s];
        if (t + s + kPF < t1) load(f[s], sb[s], sa[s], t + s + kPF);
        acc = mfma_fp6<FB, FA, 0, 0>(b0, a0, acc, csb, csa);
        acc = mfma_fp6<FB, FA, 1, 1>(b1, a1, acc, csb, csa);
      }
    }
  }

  // sum the 16 K-slices: register e of lane l is C[m = l % 32][n = 8*(e/4) + 4*(l/32) + e%4]
#pragma unroll
  for (int e = 0; e < 16; e++) part[wave][e][lane] = acc[e];
  __syncthreads();
  const int e = tid >> 6;  // 1024 threads = 16 registers x 64 lanes
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < kSkinnyWaves; w++) s += part[w][e][lane];
  const int m = lane & 31;
  const long nn = (long)blockIdx.x * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
  if (m < M && nn < N) store1(C + (long)m * N + nn, s);
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
