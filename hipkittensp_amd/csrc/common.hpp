// Shared device/host helpers for the MXFP6 GEMM kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mxfp6 {

typedef int v12i __attribute__((ext_vector_type(12)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define MXFP6_LDS __attribute__((address_space(3)))

// Output element traits: the kernels are instantiated for bf16 (the operator) and float (the
// unrounded accumulators, used to state the accuracy contract before the bf16 rounding).
struct OutBf16 { typedef uint16_t type; };
struct OutF32 { typedef float type; };
struct OutFp6 { typedef uint8_t type; };  // C re-quantised to MXFP6: packed [M, 3N/4] + E8M0 [M, N/32] (tiled kernel only)

// E8M0 byte of a 32-block with largest magnitude amax (floor(log2(amax)) - emax, clamped; 0 for an all-zero block)
__device__ __forceinline__ int e8m0_of_amax(float amax, int emax) {
  if (!(amax > 0.f)) return 0;
  const uint32_t u = __float_as_uint(amax);
  const int be = (int)(u >> 23);
  const int fl = be ? be - 127 : (31 - __clz((int)u)) - 149;  // fp32 subnormals included
  const int sb = fl - emax + 127;
  return sb < 0 ? 0 : (sb > 254 ? 254 : sb);
}

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 v = {lo, hi};
  bf2 r = __builtin_convertvector(v, bf2);
  return __builtin_bit_cast(uint32_t, r);
}

// Store 4 consecutive outputs (n .. n+3) of one row.
__device__ __forceinline__ void store4(uint16_t* p, float a, float b, float c, float d) {
  u32x2 v = {pack_bf16x2(a, b), pack_bf16x2(c, d)};
  *reinterpret_cast<u32x2*>(p) = v;
}
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
  v4f v = {a, b, c, d};
  *reinterpret_cast<v4f*>(p) = v;
}
__device__ __forceinline__ void store1(uint16_t* p, float a) { *p = (uint16_t)(pack_bf16x2(a, 0.f) & 0xffffu); }
__device__ __forceinline__ void store1(float* p, float a) { *p = a; }

// Optional work fused into every kernel's epilogue, in fp32 before the output rounding:
//   y = act(acc * row_scale[m] * col_scale[n] + bias[n])        (each factor / term only if its pointer is set)
// act: 0 none, 1 relu, 2 gelu (erf form), 3 silu.  bias is float or bf16 (bias_bf16).
struct Epilogue {
  const void* bias = nullptr;
  const float* row_scale = nullptr;
  const float* col_scale = nullptr;
  int bias_bf16 = 0;
  int act = 0;
};
__host__ __device__ __forceinline__ bool epilogue_any(const Epilogue& e) { return e.bias || e.row_scale || e.col_scale || e.act; }
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
// The activations in a handful of instructions each (they are unrolled over every accumulator of a tile):
// silu with the hardware exp2 / reciprocal (~1e-6 relative); gelu's erf by Abramowitz & Stegun 7.1.26
// (|error| <= 1.5e-7 absolute).
__device__ __forceinline__ float act_relu(float y) { return y > 0.f ? y : 0.f; }
__device__ __forceinline__ float act_silu(float y) { return y * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * y)); }
__device__ __forceinline__ float act_gelu(float y) {
  const float z = fabsf(y) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.f));
  const float poly = t * fmaf(t, fmaf(t, fmaf(t, fmaf(t, 1.061405429f, -1.453152027f), 1.421413741f), -0.284496736f), 0.254829592f);
  const float erf_abs = 1.f - poly * __builtin_amdgcn_exp2f(-1.4426950408889634f * z * z);
  return 0.5f * y * (1.f + copysignf(erf_abs, y));
}
__device__ __forceinline__ float epilogue_act(float y, int act) {
  if (act == 1) return act_relu(y);
  if (act == 2) return act_gelu(y);
  if (act == 3) return act_silu(y);
  return y;
}
// one element; m < M and n < N are the caller's business
__device__ __forceinline__ float epilogue_apply(const Epilogue& e, float v, long m, long n) {
  if (e.row_scale) v *= e.row_scale[m];
  if (e.col_scale) v *= e.col_scale[n];
  if (e.bias) v += e.bias_bf16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(e.bias)[n]) : reinterpret_cast<const float*>(e.bias)[n];
  return epilogue_act(v, e.act);
}

// Raw buffer resource over [base, base + bytes): out-of-range lanes of a buffer load read 0.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// D(32x32, fp32) += SA(32 x 64) . SB(32 x 64)^T with per-lane E8M0 block scales.
//   lane l supplies row l%32, K-block l/32 (32 fp6 values = 6 dwords) of each source;
//   result register v of lane l is D[8*(v/4) + 4*(l/32) + v%4][l%32]   (row from SA, column from SB).
//   OPA/OPB select which byte of the scale dword is used.
template <int FMT_SA, int FMT_SB, int OPA, int OPB>
__device__ __forceinline__ v16f mfma_fp6(v8i sa, v8i sb, v16f acc, int scale_sa, int scale_sb) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(sa, sb, acc, FMT_SA, FMT_SB, OPA, scale_sa, OPB, scale_sb);
}

// Workgroup -> output tile of the LDS-tiled kernels.  Workgroup `bid` of a launch works on tiles bid, bid + grid, ... of a
// logical order in which the round-robin placement of workgroups on the 8 XCDs (workgroup b runs on XCD b % 8) is
// undone, so that each XCD gets a contiguous run of logical tiles (xcd_remap; the idea of chiplet_transform_chunked,
// include/common/util.cuh:78-101, as an exact bijection for any tile count), and the raster walks group_m tile rows at a
// time down the columns (analysis/bf16_gemm/mi325x/kernel_8192.cpp:45-61): the tiles an XCD works on at once share
// operand rows in its L2.  Returns pm | pn << 16, or -1 past the last tile.
__host__ __device__ __forceinline__ int tile_order(int bid, int tiles_m, int tiles_n, int group_m, int xcd_remap) {
  const int nb = tiles_m * tiles_n;
  if (bid >= nb) return -1;
  int L = bid;
  if (xcd_remap) {
    const int xcd = bid & 7, idx = bid >> 3;
    const int per = nb >> 3, rem = nb & 7;
    L = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
  }
  const int width = group_m * tiles_n, group = L / width, first = group * group_m;
  const int gsz = tiles_m - first < group_m ? tiles_m - first : group_m, in = L - group * width;
  return (first + in % gsz) | (in / gsz) << 16;
}

// K split between workgroups: position of workgroup `bid` (of `total` = tiles x shares) in share-major order, share s of
// tile i at s * tiles + i.  The hardware deals workgroups to the eight XCDs round-robin; this hands XCD x the x-th
// eighth of that order, so that with eight shares or more an XCD's workgroups all work on the same K range: they pull
// that eighth of A and of B through the XCD's L2 once, where tile-by-tile order has every XCD fetch all of A for its
// tiles (256 x 8192 x 28672, eight shares: 263 MB of L2 misses for 189 MB of operands; A alone is 5.5 MB against 4 MB
// of L2).  With fewer shares an XCD gets part of one share's tiles, the same volume as before.  A bijection on
// [0, total) when total % 8 == 0; the identity otherwise, with the remap switched off (xcd_remap 0) or with xcd_remap 2
// (measurement: tile-by-tile order, XCDs dealt by tile_order).
__host__ __device__ __forceinline__ bool ksplit_by_share(int total, int xcd_remap) { return xcd_remap == 1 && (total & 7) == 0; }
__host__ __device__ __forceinline__ int ksplit_order(int bid, int total, int xcd_remap) {
  return ksplit_by_share(total, xcd_remap) ? (bid & 7) * (total >> 3) + (bid >> 3) : bid;
}

// Byte offset, inside a tile-major operand, of byte `b` (0 .. 3K/4) of row `row`; nkt = K / 128.
// Tiles are 32 rows x 96 bytes in the kernels' LDS image order (16-byte pieces, pairs swapped in
// rows with bit 3 set).
__host__ __device__ __forceinline__ size_t tile_major_offset(int row, int b, int nkt) {
  const int kt = b / 96, in = b - kt * 96, c = in >> 4, r = row & 31;
  return ((size_t)(row >> 5) * nkt + kt) * 3072 + (size_t)((r * 6 + (c ^ ((r >> 3) & 1))) * 16 + (in & 15));
}

// Byte offset, inside tile-major scales, of the E8M0 byte of K-block kb (32 elements) of row `row`; nk4 =
// ceil(K / 512).  The 16 scale bytes one row has for four K-tiles stay together, and the 32 rows of a row-tile
// are adjacent: 512-byte chunk (rt, g) at ((rt * nk4) + g) * 512, row r of the tile at r * 16 inside it.
__host__ __device__ __forceinline__ size_t tile_major_scale_offset(int row, int kb, int nk4) {
  return ((size_t)(row >> 5) * nk4 + (kb >> 4)) * 512 + (size_t)((row & 31) * 16 + (kb & 15));
}

}  // namespace mxfp6
