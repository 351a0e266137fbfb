// Generic MXFP6 GEMM: one wavefront per 32x32 output tile, operands read straight from global
// memory into the MFMA source registers.  Handles every legal shape (any M, N; K % 32 == 0); it is
// the fallback for shapes the LDS-tiled kernel does not take and an independent second
// implementation for the parity tests.  Role in the reference: the naive one-tile-per-block GEMM
// micro (kernels/gemm/bf16fp32/archive/micros/transpose_matmul/256_256_64_16.cpp:34-84).
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

template <int FA, int FB, typename Out>
__global__ __launch_bounds__(64) void gemm_generic_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                          const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bs,
                                                          typename Out::type* __restrict__ C, int M, int N, int K, int layout_a,
                                                          int layout_b, const Epilogue ep) {
  const int lane = threadIdx.x, h = lane >> 5, r = lane & 31;
  // tile rows beyond the 65535 a grid dimension holds continue in blockIdx.z
  const long m = ((long)blockIdx.z * 65535 + blockIdx.y) * 32 + r, n = (long)blockIdx.x * 32 + r;
  if (m - r >= M) return;
  const int nkb = K / 32;
  const long rowbytes = (long)nkb * 24;
  const bool mv = m < M, nv = n < N;
  const uint32_t* arow = reinterpret_cast<const uint32_t*>(A + (mv ? m : 0) * rowbytes);
  const uint32_t* brow = reinterpret_cast<const uint32_t*>(B + (nv ? n : 0) * rowbytes);
  const uint8_t* asr = As + (mv ? m : 0) * nkb;
  const uint8_t* bsr = Bs + (nv ? n : 0) * nkb;
  v16f acc;
  for (int i = 0; i < 16; i++) acc[i] = 0.f;
  for (int kb0 = 0; kb0 < nkb; kb0 += 2) {
    const int kb = kb0 + h;
    const bool kv = kb < nkb;
    v8i a = {0, 0, 0, 0, 0, 0, 0, 0}, b = {0, 0, 0, 0, 0, 0, 0, 0};
    int sa = 127, sb = 127;
    if (kv && mv) {
      for (int i = 0; i < 6; i++)
        a[i] = layout_a ? *reinterpret_cast<const int*>(A + tile_major_offset((int)m, kb * 24 + 4 * i, nkb / 4)) : (int)arow[kb * 6 + i];
      sa = layout_a ? As[tile_major_scale_offset((int)m, kb, (nkb + 15) / 16)] : asr[kb];
    }
    if (kv && nv) {
      for (int i = 0; i < 6; i++)
        b[i] = layout_b ? *reinterpret_cast<const int*>(B + tile_major_offset((int)n, kb * 24 + 4 * i, nkb / 4)) : (int)brow[kb * 6 + i];
      sb = layout_b ? Bs[tile_major_scale_offset((int)n, kb, (nkb + 15) / 16)] : bsr[kb];
    }
    // rows of the first source index n (B), columns index m (A): each lane then owns 4 consecutive n
    acc = mfma_fp6<FB, FA, 0, 0>(b, a, acc, sb, sa);
  }
  if (!mv) return;
  typename Out::type* crow = C + m * (long)N;
  const long n0 = (long)blockIdx.x * 32 + 4 * h;
  const bool has_ep = epilogue_any(ep);
  for (int g = 0; g < 4; g++)
    for (int e = 0; e < 4; e++) {
      long nn = n0 + 8 * g + e;
      if (nn < N) store1(crow + nn, has_ep ? epilogue_apply(ep, acc[4 * g + e], m, nn) : acc[4 * g + e]);
    }
}

template <int FA, int FB, typename Out>
static hipError_t launch(const GemmArgs& g, hipStream_t s) {
  const unsigned tm = (g.M + 31) / 32;
  dim3 grid((g.N + 31) / 32, tm < 65535 ? tm : 65535, (tm + 65534) / 65535);
  gemm_generic_kernel<FA, FB, Out><<<grid, 64, 0, s>>>(g.A, g.B, g.As, g.Bs, (typename Out::type*)g.C, g.M, g.N, g.K, g.layout_a, g.layout_b, g.ep);
  return hipGetLastError();
}

hipError_t launch_gemm_generic(const GemmArgs& g, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (g.fmt_a == FA && g.fmt_b == FB) return g.f32out ? launch<FA, FB, OutF32>(g, s) : launch<FA, FB, OutBf16>(g, s);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipErrorInvalidValue;
}

}  // namespace mxfp6
