// fp32 -> MXFP6 quantise + pack on the GPU, and the zero fill used for K == 0.
// One lane handles one 32-element block: 128 bytes in (8 x 16-byte loads), 24 bytes + 1 scale byte out.
// HBM-bound elementwise work: 4 B/element read, 0.78 B/element written.
#include "common.hpp"
#include "kernels.hpp"

namespace mxfp6 {

// Round a non-negative, already scaled magnitude to the fp6 grid (ties to even, saturating) with
// integer arithmetic on the fp32 bits.  MB = mantissa bits, BIAS = exponent bias, EB = exponent bits.
template <int MB, int BIAS, int EB>
__device__ __forceinline__ uint32_t quantise_mag(float a) {
  const uint32_t u = __float_as_uint(a);
  if (a != a) return 31u;
  const int be = (int)(u >> 23);
  if (be == 0) return 0u;  // fp32 subnormal: far below half of the smallest fp6 step
  const int ex = be - 127;
  constexpr int emin = 1 - BIAS;
  const int e = ex < emin ? emin : ex;
  const int shift = 23 - MB + (e - ex);
  uint32_t q = 0;
  if (shift < 32) {
    const uint32_t man = (u & 0x7FFFFFu) | 0x800000u;
    const uint32_t half = 1u << (shift - 1), frac = man & ((half << 1) - 1);
    q = man >> shift;
    q += (frac > half || (frac == half && (q & 1u))) ? 1u : 0u;
  }
  uint32_t code;
  if (ex < emin) {
    code = q;  // subnormal (q == 2^MB lands on the smallest normal)
  } else {
    int ee = e;
    if (q == (2u << MB)) { q = 1u << MB; ee += 1; }
    code = ((uint32_t)(ee + BIAS) << MB) | (q - (1u << MB));
    if (ee + BIAS >= (1 << EB)) code = 31u;
  }
  return code > 31u ? 31u : code;
}

template <int FMT>
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ X, uint8_t* __restrict__ packed,
                                                       uint8_t* __restrict__ scales, long nblocks, int nkb, int layout) {
  constexpr int MB = FMT == 2 ? 3 : 2, BIAS = FMT == 2 ? 1 : 3, EB = FMT == 2 ? 2 : 3, EMAX = FMT == 2 ? 2 : 4;
  const long b = (long)blockIdx.x * 256 + threadIdx.x;
  if (b >= nblocks) return;
  const v4f* src = reinterpret_cast<const v4f*>(X + b * 32);
  v4f x[8];
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = src[i];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) amax = fmaxf(amax, fabsf(x[i][j]));
  int sb = 0;
  if (amax > 0.f) {
    const uint32_t u = __float_as_uint(amax);
    const int be = (int)(u >> 23);
    const int fl = be ? be - 127 : (31 - __clz((int)u)) - 149;  // floor(log2(amax)), fp32 subnormals included
    sb = fl - EMAX + 127;
    sb = sb < 0 ? 0 : (sb > 254 ? 254 : sb);
  }
  // multiply by 2^(127 - sb) exactly: split the power of two so that each factor is a normal fp32
  const int ex = 127 - sb;  // in [-127, 127]
  const float f1 = __uint_as_float((uint32_t)((ex / 2) + 127) << 23);
  const float f2 = __uint_as_float((uint32_t)((ex - ex / 2) + 127) << 23);
  uint32_t w[6] = {0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 8; i++) {
    uint32_t g = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float v = x[i][j];
      const float y = fabsf(v) * f1 * f2;
      const uint32_t code = quantise_mag<MB, BIAS, EB>(y) | ((__float_as_uint(v) >> 31) << 5);
      g |= code << (6 * j);
    }
    // group i is 24 bits at bit 24*i of the 192-bit block
    const int bit = 24 * i, d = bit >> 5, sh = bit & 31;
    w[d] |= g << sh;
    if (sh > 8) w[d + 1] |= g >> (32 - sh);
  }
  if (layout == 0) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(packed + b * 24);
#pragma unroll
    for (int i = 0; i < 6; i++) dst[i] = w[i];
  } else {
    const int row = (int)(b / nkb), kb = (int)(b - (long)row * nkb);
#pragma unroll
    for (int i = 0; i < 6; i++) *reinterpret_cast<uint32_t*>(packed + tile_major_offset(row, kb * 24 + 4 * i, nkb / 4)) = w[i];
    scales[tile_major_scale_offset(row, kb, (nkb + 15) / 16)] = (uint8_t)sb;
    return;
  }
  scales[b] = (uint8_t)sb;
}

hipError_t launch_quantize(const float* X, uint8_t* packed, uint8_t* scales, int rows, int K, int fmt, int layout, hipStream_t s) {
  const long nblocks = (long)rows * (K / 32);
  const unsigned grid = (unsigned)((nblocks + 255) / 256);
  if (fmt == 2)
    quantize_kernel<2><<<grid, 256, 0, s>>>(X, packed, scales, nblocks, K / 32, layout);
  else
    quantize_kernel<3><<<grid, 256, 0, s>>>(X, packed, scales, nblocks, K / 32, layout);
  return hipGetLastError();
}

// row-major <-> tile-major: one lane moves one 16-byte piece
__global__ __launch_bounds__(256) void tile_operand_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, long npieces,
                                                          int nkt, int tile) {
  const long s = (long)blockIdx.x * 256 + threadIdx.x;
  if (s >= npieces) return;
  // s indexes the row-major pieces: row = s / (6 nkt), piece p of the row
  const int per_row = 6 * nkt;
  const int row = (int)(s / per_row), p = (int)(s - (long)row * per_row);
  const size_t rm = (size_t)s * 16, tm = tile_major_offset(row, p * 16, nkt);
  const v4i v = *reinterpret_cast<const v4i*>(src + (tile ? rm : tm));
  *reinterpret_cast<v4i*>(dst + (tile ? tm : rm)) = v;
}

hipError_t launch_tile_operand(const uint8_t* src, uint8_t* dst, int rows, int K, int tile, hipStream_t s) {
  const long npieces = (long)rows * (K / 128) * 6;
  if (npieces == 0) return hipSuccess;
  tile_operand_kernel<<<(unsigned)((npieces + 255) / 256), 256, 0, s>>>(src, dst, npieces, K / 128, tile);
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
