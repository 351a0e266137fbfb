// Measurement probes (no counterpart in the reference): what the silicon sustains on the two resources the GEMM
// kernels are priced against, measured with the caller's own operand bytes.
//
//   mfma_probe_kernel    every wave keeps two fragments of A and two of B (real packed fp6 rows and their E8M0 bytes,
//                        fetched once) in registers and issues nothing but v_mfma_scale_f32_32x32x64_f8f6f4 on four
//                        independent accumulators: the rate at which the matrix cores run on these bits once every
//                        other unit is idle.  The shader clock falls under such a load (the chip is power-managed), so
//                        the kernel also reports the clocks it ran for (s_memtime) against real time (s_memrealtime,
//                        100 MHz).
//   stream_probe_kernel  every wave streams a private contiguous region of a buffer through direct-to-LDS loads, 16 KB
//                        in flight per wave, no arithmetic: the read rate of a kernel that does nothing else.
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

namespace {

__device__ __forceinline__ void stamp(uint32_t* dst) {
  uint64_t t, r;
  asm volatile("s_memtime %0\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)" : "=s"(t), "=s"(r)::"memory");
  dst[0] = (uint32_t)t, dst[1] = (uint32_t)r;
}

}  // namespace

// stats[0..3] = shader clock / real-time counter at the start and at the end of workgroup 0
template <int FA, int FB>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ Bs, int rows_a, int rows_b, int K, int iters, float* sink,
                                                         uint32_t* stats) {
  const int lane = threadIdx.x & 63, gw = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int r = lane & 31, kb = lane >> 5, nkb = K / 32;
  v8i a[2], b[2];
  int sa[2], sb[2];
#pragma unroll
  for (int q = 0; q < 2; q++) {
    const long ra = (long)((gw * 2 + q) * 32 + r) % rows_a, rb = (long)((gw * 2 + q) * 32 + r) % rows_b;
    const int k = ((gw + q) * 2 + kb) % nkb;
    const uint32_t* pa = reinterpret_cast<const uint32_t*>(A + ra * (nkb * 24) + k * 24);
    const uint32_t* pb = reinterpret_cast<const uint32_t*>(B + rb * (nkb * 24) + k * 24);
    a[q] = v8i{0, 0, 0, 0, 0, 0, 0, 0}, b[q] = v8i{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 6; i++) a[q][i] = (int)pa[i], b[q][i] = (int)pb[i];
    sa[q] = As[ra * nkb + k], sb[q] = Bs[rb * nkb + k];
  }
  v16f acc[4];
#pragma unroll
  for (int n = 0; n < 4; n++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[n][i] = 0.f;
  if (blockIdx.x == 0 && threadIdx.x == 0) stamp(stats);
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int n = 0; n < 4; n++) acc[n] = mfma_fp6<FB, FA, 0, 0>(b[n >> 1], a[n & 1], acc[n], sb[n >> 1], sa[n & 1]);
  }
  float s = 0.f;
#pragma unroll
  for (int n = 0; n < 4; n++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[n][i];
  if (blockIdx.x == 0 && threadIdx.x == 0) stamp(stats + 2);
  if (s == 1.2345e-30f) sink[0] = s;  // keeps the accumulators alive
}

hipError_t launch_mfma_probe(const uint8_t* A, const uint8_t* B, const uint8_t* As, const uint8_t* Bs, int rows_a, int rows_b, int K, int fmt_a,
                             int fmt_b, int iters, int workgroups, float* sink, uint32_t* stats, hipStream_t s) {
#define MXFP6_CASE(FA, FB) \
  if (fmt_a == FA && fmt_b == FB) mfma_probe_kernel<FA, FB><<<workgroups, 256, 0, s>>>(A, B, As, Bs, rows_a, rows_b, K, iters, sink, stats);
  MXFP6_CASE(2, 2) MXFP6_CASE(2, 3) MXFP6_CASE(3, 2) MXFP6_CASE(3, 3)
#undef MXFP6_CASE
  return hipGetLastError();
}

// Each of the grid's workgroups of NW waves streams bytes / gridDim.x contiguous bytes, each wave its own share of them,
// 1 KB per direct load, 16 loads in flight per wave (NW = 8: one workgroup fills a compute unit's LDS; NW = 4: two do).
template <int NW>
__global__ __launch_bounds__(NW * 64) void stream_probe_kernel(const uint8_t* __restrict__ buf, uint32_t bytes_per_wave, uint32_t* stats) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NW * 16384];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint8_t* base = buf + ((size_t)blockIdx.x * NW + wave) * bytes_per_wave;
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(base, bytes_per_wave);
  const uint32_t lds = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem + wave * 16384;
  if (blockIdx.x == 0 && threadIdx.x == 0) stamp(stats);
  const int voff = lane * 16;
  for (uint32_t off = 0; off < bytes_per_wave; off += 8192) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds + (((off >> 13) & 1) * 8 + i) * 1024);
      const int so = __builtin_amdgcn_readfirstlane((int)(off + i * 1024));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(dst), "v"(voff), "s"(rsrc), "s"(so) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // the batch before this one has landed: its half of the buffer is free again
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (blockIdx.x == 0 && threadIdx.x == 0) stamp(stats + 2);
}

hipError_t launch_stream_probe(const uint8_t* buf, size_t bytes, int workgroups, int waves, uint32_t* stats, hipStream_t s) {
  const size_t per_wave = bytes / ((size_t)workgroups * waves);
  if (per_wave == 0 || per_wave % 8192 != 0 || per_wave >= ((size_t)1 << 32)) return hipErrorInvalidValue;
  if (waves == 8) stream_probe_kernel<8><<<workgroups, 512, 0, s>>>(buf, (uint32_t)per_wave, stats);
  else if (waves == 4) stream_probe_kernel<4><<<workgroups, 256, 0, s>>>(buf, (uint32_t)per_wave, stats);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace mxfp6
