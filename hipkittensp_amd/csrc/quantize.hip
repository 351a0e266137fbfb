// fp32 -> MXFP6 quantise + pack on the GPU, the tile-major re-layout copies, and the zero fill used for K == 0.
// HBM-bound elementwise work: 4 B/element read, 0.78 B/element written.
#include "common.hpp"
#include "kernels.hpp"
#include "loader.hpp"

namespace mxfp6 {

// Quantiser.  One lane handles one 32-element block (128 bytes in, 24 bytes + 1 scale byte out), but the memory
// system wants consecutive lanes on consecutive bytes: a wave fetches 64 blocks (8 KB, contiguous) with eight
// direct-to-LDS loads of 16 bytes per lane into a private buffer and every lane reads its own block back.  The
// buffer is an image of memory with the eight 16-byte pieces of block b rotated: piece c lives in slot
// b * 8 + (c ^ (b & 7)), chosen by which global bytes each lane fetches (a direct load writes lane l at 16 l), so
// that the 16 lanes of a ds_read_b128 phase spread over all banks.  The conversion itself is the hardware's:
// v_cvt_scalef32_2xpk16_{fp6,bf6}_f32 divides 32 floats by a power of two and rounds them to e2m3 / e3m2 (nearest
// even, saturating, NaN -> largest magnitude, fp32 subnormals -> 0); its result interleaves its two sources,
// so they are the even and the odd elements of the block.  (With the rounding done by integer arithmetic, ~25
// instructions per element, the kernel was ALU-bound at 4.4 TB/s.)
// Row-major output: a wave's 64 blocks are consecutive (1536 contiguous output bytes).  Tile-major output: they are
// 16 rows x one K-tile (512 input bytes per row, four whole lines), which is half of a 3 KB output tile and again
// 1536 contiguous bytes; a block's 24 bytes are three 8-byte stores (an aligned 8-byte run never straddles the
// 16-byte pieces the tile-major order permutes).
constexpr int kQWaves = 4;  // waves per workgroup; a wave fetches 64 blocks at a time (8 KB of fp32, 4 KB of bf16)


// In: float, or uint16_t for bf16 (the same values after the exact widening: the bf16 instruction
// v_cvt_scalef32_pk32_{fp6,bf6}_bf16 was checked against the fp32 one on 1 M values per format, no difference).
template <int FMT, typename In>
__global__ __launch_bounds__(kQWaves * 64) void quantize_kernel(const In* __restrict__ X, uint8_t* __restrict__ packed,
                                                              uint8_t* __restrict__ scales, long nblocks, int nkb, int layout) {
  constexpr int EMAX = FMT == 2 ? 2 : 4;
  constexpr int BB = 32 * (int)sizeof(In), P = BB / 16;  // bytes and 16-byte pieces of a block
  constexpr int kChunk = 64 * BB, NLD = kChunk / 1024;   // bytes and direct loads of a chunk
  __shared__ __attribute__((aligned(1024))) uint8_t smem[kQWaves * kChunk];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t buf = (uint32_t)(uintptr_t)(MXFP6_LDS uint8_t*)smem + wave * kChunk;
  const long nchunks = (nblocks + 63) / 64;
  const long stride = (long)gridDim.x * kQWaves;
  long chunk = (long)blockIdx.x * kQWaves + wave;
  const int nkt = nkb / 4;  // tile-major only: K-tiles per row

  // slot s = q * 64 + lane of load q holds piece (s % P) ^ (b % P) of the chunk's block b = s / P; tile-major:
  // block b is K-block b % 4 of row b / 4 of the chunk
  int voff[NLD];
#pragma unroll
  for (int q = 0; q < NLD; q++) {
    const int sl = q * 64 + lane, b = sl / P, c = (sl % P) ^ (b % P);
    voff[q] = layout ? (b >> 2) * (nkb * BB) + (b & 3) * BB + c * 16 : (b * P + c) * 16;
  }
  auto fetch = [&](long ch) __attribute__((always_inline)) {
    // the resource covers this chunk only (the whole input may exceed 4 GB); bytes past the end read as zero
    if (layout) {
      const long g16 = ch / nkt, kt = ch - g16 * nkt;
      const __amdgpu_buffer_rsrc_t r = make_rsrc(reinterpret_cast<const uint8_t*>(X) + (g16 * 16 * nkb + kt * 4) * BB, (uint32_t)(15 * nkb * BB + 4 * BB));
#pragma unroll
      for (int q = 0; q < NLD; q++) dma16(r, buf + q * 1024, voff[q], 0);
    } else {
      const long left = nblocks * BB - ch * kChunk;
      const __amdgpu_buffer_rsrc_t r = make_rsrc(reinterpret_cast<const uint8_t*>(X) + ch * kChunk, (uint32_t)(left < kChunk ? left : kChunk));
#pragma unroll
      for (int q = 0; q < NLD; q++) dma16(r, buf + q * 1024, voff[q], 0);
    }
  };
  if (chunk < nchunks) fetch(chunk);
  for (; chunk < nchunks; chunk += stride) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    v4i x[P];
#pragma unroll
    for (int c = 0; c < P; c++) x[c] = *reinterpret_cast<const v4i*>(smem + wave * kChunk + lane * BB + ((c ^ (lane % P)) * 16));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (chunk + stride < nchunks) fetch(chunk + stride);  // the buffer is free again: the next chunk streams in under the arithmetic

    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < P; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        if constexpr (sizeof(In) == 4) {
          amax = fmaxf(amax, fabsf(__int_as_float(x[i][j])));
        } else {
          amax = fmaxf(amax, fabsf(__int_as_float(x[i][j] << 16)));
          amax = fmaxf(amax, fabsf(__int_as_float(x[i][j] & (int)0xffff0000)));
        }
      }
    int sb = 0;
    if (amax > 0.f) {
      const uint32_t u = __float_as_uint(amax);
      const int be = (int)(u >> 23);
      const int fl = be ? be - 127 : (31 - __clz((int)u)) - 149;  // floor(log2(amax)), fp32 subnormals included
      sb = fl - EMAX + 127;
      sb = sb < 0 ? 0 : (sb > 254 ? 254 : sb);
    }
    const float scale = __uint_as_float((uint32_t)sb << 23);  // 2^(sb - 127); the instruction uses the exponent field
    typedef unsigned v6u __attribute__((ext_vector_type(6)));
    v6u w;
    if constexpr (sizeof(In) == 4) {
      v16f ev, od;
#pragma unroll
      for (int i = 0; i < 16; i++) ev[i] = __int_as_float(x[i / 2][(2 * i) & 3]), od[i] = __int_as_float(x[i / 2][(2 * i + 1) & 3]);
      if constexpr (FMT == 2) w = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(ev, od, scale);
      else w = __builtin_amdgcn_cvt_scalef32_2xpk16_bf6_f32(ev, od, scale);
    } else {
      typedef __bf16 v32bf __attribute__((ext_vector_type(32)));
      typedef int v16i __attribute__((ext_vector_type(16)));
      v16i raw;
#pragma unroll
      for (int i = 0; i < 16; i++) raw[i] = x[i / 4][i & 3];
      const v32bf xb = __builtin_bit_cast(v32bf, raw);
      if constexpr (FMT == 2) w = __builtin_amdgcn_cvt_scalef32_pk32_fp6_bf16(xb, scale);
      else w = __builtin_amdgcn_cvt_scalef32_pk32_bf6_bf16(xb, scale);
    }
    if (layout == 0) {
      const long b = chunk * 64 + lane;
      if (b >= nblocks) continue;
      u32x2* dst = reinterpret_cast<u32x2*>(packed + b * 24);
#pragma unroll
      for (int i = 0; i < 3; i++) dst[i] = u32x2{w[2 * i], w[2 * i + 1]};
      scales[b] = (uint8_t)sb;
    } else {
      const long g16 = chunk / nkt;
      const int kt = (int)(chunk - g16 * nkt);
      const int row = (int)(g16 * 16) + (lane >> 2), kb = kt * 4 + (lane & 3);
#pragma unroll
      for (int i = 0; i < 3; i++)
        *reinterpret_cast<u32x2*>(packed + tile_major_offset(row, kb * 24 + 8 * i, nkt)) = u32x2{w[2 * i], w[2 * i + 1]};
      scales[tile_major_scale_offset(row, kb, (nkb + 15) / 16)] = (uint8_t)sb;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

hipError_t launch_quantize(const void* X, int x_bf16, uint8_t* packed, uint8_t* scales, int rows, int K, int fmt, int layout, hipStream_t s) {
  const long nblocks = (long)rows * (K / 32);
  if (nblocks == 0) return hipSuccess;
  const long nchunks = (nblocks + 63) / 64, want = (nchunks + kQWaves - 1) / kQWaves;
  const unsigned grid = (unsigned)(want < 256 * 5 ? want : 256 * 5);  // five workgroups of 32 KB LDS fit a CU
#define MXFP6_Q(FMT, T) quantize_kernel<FMT, T><<<grid, kQWaves * 64, 0, s>>>((const T*)X, packed, scales, nblocks, K / 32, layout)
  if (fmt == 2) { if (x_bf16) MXFP6_Q(2, uint16_t); else MXFP6_Q(2, float); }
  else { if (x_bf16) MXFP6_Q(3, uint16_t); else MXFP6_Q(3, float); }
#undef MXFP6_Q
  return hipGetLastError();
}

// row-major <-> tile-major.  A workgroup moves 32 rows x four K-tiles: 384 row-major bytes per row (three whole cache
// lines) against four whole 3 KB tiles, so both sides are touched in whole lines by one workgroup (one 16-byte piece
// per lane in row-major order over the whole operand ran at 3.9 TB/s, this at 5.8).
__global__ __launch_bounds__(256) void tile_operand_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int nkt, int nk4,
                                                          int tile) {
  const int rt = blockIdx.x / nk4, g = blockIdx.x - rt * nk4;  // row-tile, group of four K-tiles
  const int ntile = min(4, nkt - 4 * g);
  const size_t rm0 = ((size_t)rt * 32 * nkt + 4 * g) * 96, tm0 = ((size_t)rt * nkt + 4 * g) * 3072;
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int p = threadIdx.x + 256 * i, r = p / 24, q = p - r * 24;  // piece q of the row's 384 bytes
    const int tg = q / 6, c = q - tg * 6;
    if (tg >= ntile) continue;
    const size_t rm = rm0 + (size_t)r * nkt * 96 + q * 16, tm = tm0 + tg * 3072 + (r * 6 + (c ^ ((r >> 3) & 1))) * 16;
    *reinterpret_cast<v4i*>(dst + (tile ? tm : rm)) = *reinterpret_cast<const v4i*>(src + (tile ? rm : tm));
  }
}

hipError_t launch_tile_operand(const uint8_t* src, uint8_t* dst, int rows, int K, int tile, hipStream_t s) {
  const int nkt = K / 128, nk4 = (nkt + 3) / 4;
  const long blocks = (long)(rows / 32) * nk4;
  if (blocks == 0) return hipSuccess;
  tile_operand_kernel<<<(unsigned)blocks, 256, 0, s>>>(src, dst, nkt, nk4, tile);
  return hipGetLastError();
}

// scales [rows, K/32] row-major <-> tile-major: one lane moves the (up to) 16 bytes one row has for four K-tiles;
// K-blocks past K (K % 512 != 0) are written as zero in the tile-major direction
__global__ __launch_bounds__(256) void tile_scales_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, long nchunks,
                                                         int nkb, int nk4, int tile) {
  const long s = (long)blockIdx.x * 256 + threadIdx.x;
  if (s >= nchunks) return;
  const int row = (int)(s / nk4), g = (int)(s - (long)row * nk4);
  const int nvalid = min(16, nkb - g * 16);  // a multiple of 4: K % 128 == 0
  const size_t rm = (size_t)row * nkb + (size_t)g * 16, tm = tile_major_scale_offset(row, g * 16, nk4);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (tile) {
      *reinterpret_cast<uint32_t*>(dst + tm + 4 * i) = 4 * i < nvalid ? *reinterpret_cast<const uint32_t*>(src + rm + 4 * i) : 0u;
    } else if (4 * i < nvalid) {
      *reinterpret_cast<uint32_t*>(dst + rm + 4 * i) = *reinterpret_cast<const uint32_t*>(src + tm + 4 * i);
    }
  }
}

hipError_t launch_tile_scales(const uint8_t* src, uint8_t* dst, int rows, int K, int tile, hipStream_t s) {
  const int nkb = K / 32, nk4 = (nkb + 15) / 16;
  const long nchunks = (long)rows * nk4;
  if (nchunks == 0) return hipSuccess;
  tile_scales_kernel<<<(unsigned)((nchunks + 255) / 256), 256, 0, s>>>(src, dst, nchunks, nkb, nk4, tile);
  return hipGetLastError();
}

// Row-major -> tile-major for up to two operands (packed bytes and scales) in one launch: the re-layout pre-pass of
// the gemm entry points, where every extra launch would cost as much as part of the copy.  A workgroup copies 32
// rows x four K-tiles (384 source bytes per row = three whole cache lines; a single K-tile's 96 bytes straddle
// lines, and lines shared between workgroups on different XCDs were fetched twice: 1.64x read traffic) in source
// order: consecutive lanes read consecutive 16-byte pieces of a row and write runs of 96 bytes into the four 3 KB
// tiles.  Other workgroups move the 16 scale bytes one row has for four K-tiles, one row per lane.
struct TileJob {
  const uint8_t* src;
  uint8_t* dst;
  const uint8_t* ssrc;
  uint8_t* sdst;
  long ngroups, nchunks;  // groups of 32 rows x four K-tiles; (row, four K-tiles) scale chunks
  unsigned pblocks, sblocks;
};

__global__ __launch_bounds__(256) void tile_both_kernel(TileJob j0, TileJob j1, int nkt, int nkb, int nk4) {
  unsigned bid = blockIdx.x;
  const bool second = bid >= j0.pblocks + j0.sblocks;
  if (second) bid -= j0.pblocks + j0.sblocks;
  const TileJob& j = second ? j1 : j0;
  if (bid < j.pblocks) {
    const int rt = bid / nk4, g = bid - rt * nk4;  // row-tile, group of four K-tiles
    const int ntile = min(4, nkt - 4 * g);
    const uint8_t* src = j.src + ((size_t)rt * 32 * nkt + 4 * g) * 96;
    uint8_t* dst = j.dst + ((size_t)rt * nkt + 4 * g) * 3072;
#pragma unroll
    for (int i = 0; i < 3; i++) {
      const int p = threadIdx.x + 256 * i, r = p / 24, q = p - r * 24;  // piece q of the row's 384 bytes
      const int tg = q / 6, c = q - tg * 6;
      if (tg < ntile)
        *reinterpret_cast<v4i*>(dst + tg * 3072 + (r * 6 + (c ^ ((r >> 3) & 1))) * 16) =
            *reinterpret_cast<const v4i*>(src + (size_t)r * nkt * 96 + q * 16);
    }
  } else {
    const long s = (long)(bid - j.pblocks) * 256 + threadIdx.x;
    if (s >= j.nchunks) return;
    const int row = (int)(s / nk4), g = (int)(s - (long)row * nk4);
    const int nvalid = min(16, nkb - g * 16);
    const size_t rm = (size_t)row * nkb + (size_t)g * 16, tm = tile_major_scale_offset(row, g * 16, nk4);
#pragma unroll
    for (int i = 0; i < 4; i++)
      *reinterpret_cast<uint32_t*>(j.sdst + tm + 4 * i) = 4 * i < nvalid ? *reinterpret_cast<const uint32_t*>(j.ssrc + rm + 4 * i) : 0u;
  }
}

// rows1 == 0: only the first operand
hipError_t launch_tile_both(const uint8_t* src0, uint8_t* dst0, const uint8_t* ssrc0, uint8_t* sdst0, int rows0, const uint8_t* src1,
                            uint8_t* dst1, const uint8_t* ssrc1, uint8_t* sdst1, int rows1, int K, hipStream_t s) {
  const int nkt = K / 128, nkb = K / 32, nk4 = (nkb + 15) / 16;
  auto job = [&](const uint8_t* src, uint8_t* dst, const uint8_t* ssrc, uint8_t* sdst, int rows) {
    TileJob j{src, dst, ssrc, sdst, (long)(rows / 32) * nk4, (long)rows * nk4, 0, 0};
    j.pblocks = (unsigned)j.ngroups;
    j.sblocks = (unsigned)((j.nchunks + 255) / 256);
    return j;
  };
  const TileJob j0 = job(src0, dst0, ssrc0, sdst0, rows0), j1 = job(src1, dst1, ssrc1, sdst1, rows1);
  const unsigned blocks = j0.pblocks + j0.sblocks + j1.pblocks + j1.sblocks;
  if (blocks == 0) return hipSuccess;
  tile_both_kernel<<<blocks, 256, 0, s>>>(j0, j1, nkt, nkb, nk4);
  return hipGetLastError();
}

__global__ void fill_zero_kernel(uint8_t* p, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, st = (size_t)gridDim.x * 256;
  for (; i < n; i += st) p[i] = 0;
}

hipError_t launch_fill_zero(void* p, size_t bytes, hipStream_t s) {
  size_t blocks = (bytes + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks == 0) return hipSuccess;
  fill_zero_kernel<<<(unsigned)blocks, 256, 0, s>>>((uint8_t*)p, bytes);
  return hipGetLastError();
}

}  // namespace mxfp6
