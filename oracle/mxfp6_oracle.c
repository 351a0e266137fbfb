/*
 * CPU oracle (plain C) for the MXFP6 block-scaled GEMM path -- TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * Linked/loaded only by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
 *
 * The reference tree holds no FP6 source (its FP6 GEMM is on an unmounted branch,
 * kernels/gemm/README.md:6-7), so this restates the contract of BASELINE.json configs[0]
 * (per-32 E8M0 scale 2^(floor(log2(blockmax)) - emax), fp6 round-to-nearest-even, dense
 * 4-values-per-3-bytes packing, C = A . B^T with fp32 accumulation, bf16 output) with the OCP MX
 * v1.0 closed forms.  Structure follows the reference's host oracles:
 *   C = A . B^T triple loop          tests/unit/warp/register/tile/mma.cu:44-55
 *   both operands K-contiguous       kernels/gemm/bf16fp32/utils.py:28-37
 *   seeded host init + timing shape  kernels/gemm/fp8fp32/profile_utils.cpp:5-45
 *
 * This file is written independently of oracle/mxfp6_oracle.py (bit manipulation here, frexp /
 * ldexp arithmetic there); tests/test_oracle.py requires the two to agree bit for bit, and
 * each is separately pinned against closed forms, brute force and the golden vectors under
 * tests/golden/.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define MXFP6_E2M3 2
#define MXFP6_E3M2 3

static int fmt_mbits(int fmt) { return fmt == MXFP6_E2M3 ? 3 : 2; }
static int fmt_ebits(int fmt) { return fmt == MXFP6_E2M3 ? 2 : 3; }
static int fmt_bias(int fmt) { return fmt == MXFP6_E2M3 ? 1 : 3; }
static int fmt_emax(int fmt) { return fmt == MXFP6_E2M3 ? 2 : 4; }

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp6 code -> fp32, built from the bit fields (no table lookup, no libm). */
float mxfp6o_decode(int fmt, int code) {
  int mb = fmt_mbits(fmt), bias = fmt_bias(fmt);
  int s = (code >> 5) & 1, e = (code >> mb) & ((1 << fmt_ebits(fmt)) - 1), m = code & ((1 << mb) - 1);
  float v;
  if (e == 0) {
    v = (float)m;                      /* m * 2^(1 - bias - mb) */
    for (int i = 0; i < bias - 1 + mb; i++) v *= 0.5f;
  } else {
    /* assemble the IEEE-754 single directly: exponent e - bias + 127, mantissa m << (23 - mb) */
    v = u2f(((uint32_t)(e - bias + 127) << 23) | ((uint32_t)m << (23 - mb)));
  }
  return s ? -v : v;
}

void mxfp6o_decode_table(int fmt, float *out64) {
  for (int c = 0; c < 64; c++) out64[c] = mxfp6o_decode(fmt, c);
}

/* E8M0 byte -> fp32 2^(b-127); 255 -> NaN; 0 -> 2^-127 (subnormal fp32). */
float mxfp6o_e8m0(int b) {
  if (b == 255) return u2f(0x7FC00000u);
  if (b == 0) return u2f(0x00400000u);
  return u2f((uint32_t)b << 23);
}

/* Round a non-negative scaled magnitude to the fp6 grid, ties to even, saturating: integer
 * arithmetic on the fp32 bit pattern. */
static int quantise_mag(int fmt, float a) {
  int mb = fmt_mbits(fmt), bias = fmt_bias(fmt);
  int maxcode = 31; /* all exponent and mantissa bits set */
  uint32_t u = f2u(a);
  if (a != a) return maxcode;
  int ex = (int)(u >> 23) - 127;                 /* unbiased fp32 exponent */
  uint64_t man = (u & 0x7FFFFFu) | 0x800000u;    /* 1.23 significand   */
  if ((u >> 23) == 0) { return 0; }              /* fp32 subnormal: far below half the smallest fp6 step */
  int emin = 1 - bias;
  int shift;                                     /* bits to drop from the 24-bit significand */
  int e = ex;
  if (e < emin) e = emin;                        /* subnormal target binade */
  shift = 23 - mb + (e - ex);
  uint64_t q;
  if (shift >= 40) q = 0;
  else {
    uint64_t half = 1ull << (shift - 1), mask = (1ull << shift) - 1, frac = man & mask;
    q = man >> shift;
    if (frac > half || (frac == half && (q & 1))) q++;
  }
  /* q is the significand in units of 2^(e - mb): q in [0, 2^(mb+1)] */
  int code;
  if (ex < emin) {                               /* result is subnormal or the smallest normal */
    code = (int)q;                               /* q == 2^mb encodes exponent field 1, mantissa 0 */
  } else {
    if (q == (2u << mb)) { q = 1u << mb; e += 1; }
    code = ((e + bias) << mb) | (int)(q - (1u << mb));
    if (e + bias >= (1 << fmt_ebits(fmt))) code = maxcode;
  }
  if (code > maxcode) code = maxcode;
  return code;
}

/* floor(log2(x)) of a positive finite fp32, counting fp32 subnormals correctly */
static int floor_log2f(float x) {
  uint32_t u = f2u(x) & 0x7FFFFFFFu;
  int be = (int)(u >> 23);
  if (be) return be - 127;
  int p = 31 - __builtin_clz(u); /* subnormal: value = u * 2^-149 */
  return p - 149;
}

int mxfp6o_block_scale(const float *x32, int fmt) {
  float amax = 0.0f;
  for (int i = 0; i < 32; i++) { float a = fabsf(x32[i]); if (a > amax) amax = a; }
  if (amax == 0.0f) return 0;
  int e = floor_log2f(amax) - fmt_emax(fmt) + 127;
  if (e < 0) e = 0;
  if (e > 254) e = 254;
  return e;
}

/* x[rows,K] fp32 -> packed [rows, 3K/4], scales [rows, K/32] */
int mxfp6o_quantise(const float *x, long rows, long K, int fmt, uint8_t *packed, uint8_t *scales) {
  if (K % 32 || (fmt != 2 && fmt != 3)) return -1;
  long nb = K / 32;
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; r++) {
    for (long b = 0; b < nb; b++) {
      const float *xb = x + r * K + b * 32;
      int sb = mxfp6o_block_scale(xb, fmt);
      scales[r * nb + b] = (uint8_t)sb;
      uint8_t *dst = packed + r * (K / 4 * 3) + b * 24;
      double inv = ldexp(1.0, 127 - sb);
      for (int g = 0; g < 8; g++) {
        uint32_t w = 0;
        for (int j = 0; j < 4; j++) {
          float v = xb[g * 4 + j];
          float y = (float)((double)v * inv);
          int code = quantise_mag(fmt, fabsf(y)) | (signbit(v) ? 32 : 0);
          w |= (uint32_t)code << (6 * j);
        }
        dst[3 * g + 0] = (uint8_t)(w & 255);
        dst[3 * g + 1] = (uint8_t)((w >> 8) & 255);
        dst[3 * g + 2] = (uint8_t)((w >> 16) & 255);
      }
    }
  }
  return 0;
}

static inline int code_at(const uint8_t *row, long j) {
  const uint8_t *p = row + (j >> 2) * 3; /* 4 codes per 3-byte group */
  uint32_t w = p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
  return (int)((w >> (6 * (j & 3))) & 63);
}

/* packed [rows, 3K/4] + scales -> out fp32 [rows, K] (ld = K), or transposed [K, rows] when transpose != 0 */
int mxfp6o_dequantise(const uint8_t *packed, const uint8_t *scales, long rows, long K, int fmt, float *out,
                      int transpose) {
  if (K % 32 || (fmt != 2 && fmt != 3)) return -1;
  float tab[64];
  mxfp6o_decode_table(fmt, tab);
  long nb = K / 32, rb = K / 4 * 3;
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; r++) {
    const uint8_t *row = packed + r * rb;
    for (long b = 0; b < nb; b++) {
      double s = ldexp(1.0, (int)scales[r * nb + b] - 127);
      for (int g = 0; g < 8; g++) {
        const uint8_t *p = row + b * 24 + g * 3;
        uint32_t w = p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
        for (int j = 0; j < 4; j++) {
          float v = (float)((double)tab[(w >> (6 * j)) & 63] * s);
          long k = b * 32 + g * 4 + j;
          if (transpose) out[k * rows + r] = v; else out[r * K + k] = v;
        }
      }
    }
  }
  return 0;
}

uint16_t mxfp6o_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if (f != f) return 0x7FC0;
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

/*
 * Dequantise-and-matmul, fp32 accumulation.  C[M,N] (fp32, ld N) = dq(A)[M,K] . dq(B)[N,K]^T.
 * A is dequantised row-major, B transposed to [K,N]; each thread owns blocks of 8 rows of C and
 * sweeps K for a 256-wide strip (i-k-j order, j vectorised by the compiler).
 * Returns 0, or -1 on bad arguments, -2 on allocation failure.
 */
int mxfp6o_gemm_f32(const uint8_t *a_packed, const uint8_t *b_packed, const uint8_t *a_scale, const uint8_t *b_scale,
                    float *C, long M, long N, long K, int fmt_a, int fmt_b) {
  if (K % 32 || M < 0 || N < 0) return -1;
  if (M == 0 || N == 0) return 0;
  float *A = (float *)malloc(sizeof(float) * (size_t)M * K);
  float *Bt = (float *)malloc(sizeof(float) * (size_t)N * K);
  if (!A || !Bt) { free(A); free(Bt); return -2; }
  if (mxfp6o_dequantise(a_packed, a_scale, M, K, fmt_a, A, 0) || mxfp6o_dequantise(b_packed, b_scale, N, K, fmt_b, Bt, 1)) {
    free(A); free(Bt); return -1;
  }
  enum { RB = 8, JB = 256 };
  long nib = (M + RB - 1) / RB, njb = (N + JB - 1) / JB;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (long ib = 0; ib < nib; ib++) {
    for (long jb = 0; jb < njb; jb++) {
      long i0 = ib * RB, i1 = i0 + RB < M ? i0 + RB : M;
      long j0 = jb * JB, jn = (j0 + JB < N ? j0 + JB : N) - j0;
      float acc[RB][JB];
      memset(acc, 0, sizeof(acc));
      for (long k = 0; k < K; k++) {
        const float *bt = Bt + k * N + j0;
        for (long i = i0; i < i1; i++) {
          float a = A[i * K + k];
          float *ac = acc[i - i0];
          for (long j = 0; j < jn; j++) ac[j] += a * bt[j];
        }
      }
      for (long i = i0; i < i1; i++) memcpy(C + i * N + j0, acc[i - i0], sizeof(float) * (size_t)jn);
    }
  }
  free(A); free(Bt);
  return 0;
}

/* Same, with the bf16 epilogue (round-to-nearest-even). */
int mxfp6o_gemm_bf16(const uint8_t *a_packed, const uint8_t *b_packed, const uint8_t *a_scale, const uint8_t *b_scale,
                     uint16_t *C, long M, long N, long K, int fmt_a, int fmt_b) {
  float *Cf = (float *)malloc(sizeof(float) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
  if (!Cf) return -2;
  int rc = mxfp6o_gemm_f32(a_packed, b_packed, a_scale, b_scale, Cf, M, N, K, fmt_a, fmt_b);
  if (!rc) for (long i = 0; i < M * N; i++) C[i] = mxfp6o_f32_to_bf16(Cf[i]);
  free(Cf);
  return rc;
}

/* fp64 brute-force triple loop for tiny shapes: the yardstick the fp32 paths are judged against. */
int mxfp6o_gemm_f64_naive(const uint8_t *a_packed, const uint8_t *b_packed, const uint8_t *a_scale,
                          const uint8_t *b_scale, double *C, long M, long N, long K, int fmt_a, int fmt_b) {
  if (K % 32) return -1;
  long rb = K / 4 * 3, nb = K / 32;
  for (long i = 0; i < M; i++)
    for (long j = 0; j < N; j++) {
      double s = 0.0;
      for (long k = 0; k < K; k++) {
        double a = (double)mxfp6o_decode(fmt_a, code_at(a_packed + i * rb, k)) * ldexp(1.0, (int)a_scale[i * nb + k / 32] - 127);
        double b = (double)mxfp6o_decode(fmt_b, code_at(b_packed + j * rb, k)) * ldexp(1.0, (int)b_scale[j * nb + k / 32] - 127);
        s += a * b;
      }
      C[i * N + j] = s;
    }
  return 0;
}

int mxfp6o_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
