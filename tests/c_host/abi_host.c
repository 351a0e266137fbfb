/*
 * A compiled caller of the C ABI with no Python and no torch in the process: what a maintainer of the reference would
 * link in place of its host launcher (analysis/bf16_gemm/mi325x/kernel_8192.cpp:227-237 builds its own pybind module
 * around such a call).  Test infrastructure: it links the product (libmxfp6_gemm.so, through include/mxfp6_gemm.h)
 * and, as the checker, the plain-C oracle (oracle/libmxfp6_oracle.so); tests/test_gpu_parity.py runs the binary that
 * the build step leaves beside this file.
 *
 * For each case: fp32 sources from a fixed generator, quantised on the host by the oracle and on the GPU by
 * mxfp6_quantize (packed bytes and scales must agree bit for bit), the product through mxfp6_gemm_f32out (metric
 * <= 2e-3 against the oracle's fp32 dequantise-and-matmul, measured before the bf16 rounding), through mxfp6_gemm
 * (its bf16 bits = round-to-nearest-even of those accumulators) and through mxfp6_gemm_noalloc (bit-identical to
 * mxfp6_gemm).  Prints one line per case and "ALL OK" at the end; the exit status is the number of failed checks.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "mxfp6_gemm.h"

/* the checker (oracle/mxfp6_oracle.c) */
int mxfp6o_quantise(const float *x, long rows, long K, int fmt, uint8_t *packed, uint8_t *scales);
int mxfp6o_gemm_f32(const uint8_t *a_packed, const uint8_t *b_packed, const uint8_t *a_scale, const uint8_t *b_scale,
                    float *C, long M, long N, long K, int fmt_a, int fmt_b);
uint16_t mxfp6o_f32_to_bf16(float f);

#define HIP_OK(call)                                                                           \
  do {                                                                                         \
    hipError_t e_ = (call);                                                                    \
    if (e_ != hipSuccess) {                                                                    \
      fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      exit(100);                                                                               \
    }                                                                                          \
  } while (0)

#define LIB_OK(call)                                                                            \
  do {                                                                                          \
    int rc_ = (call);                                                                           \
    if (rc_ != MXFP6_OK) {                                                                      \
      fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_, mxfp6_strerror(rc_)); \
      exit(101);                                                                                \
    }                                                                                           \
  } while (0)

static uint64_t g_state;
static float uniform01(void) { /* splitmix64 -> (0, 1) */
  uint64_t z = (g_state += 0x9e3779b97f4a7c15ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  z ^= z >> 31;
  return ((float)(z >> 40) + 0.5f) / 16777216.0f;
}
static void fill_normal(float *x, size_t n, float std, uint64_t seed) { /* Box-Muller */
  g_state = seed;
  for (size_t i = 0; i + 1 < n; i += 2) {
    const float r = sqrtf(-2.0f * logf(uniform01())), t = 6.2831853f * uniform01();
    x[i] = std * r * cosf(t), x[i + 1] = std * r * sinf(t);
  }
  if (n & 1) x[n - 1] = std * sqrtf(-2.0f * logf(uniform01())) * cosf(6.2831853f * uniform01());
}

static int run_case(int M, int N, int K, int fmt_a, int fmt_b, hipStream_t stream) {
  const size_t pa = (size_t)M * K / 4 * 3, pb = (size_t)N * K / 4 * 3, sa = (size_t)M * K / 32, sb = (size_t)N * K / 32;
  const size_t mn = (size_t)M * N;
  float *xa = malloc(sizeof(float) * (size_t)M * K), *xb = malloc(sizeof(float) * (size_t)N * K);
  uint8_t *ap = malloc(pa), *bp = malloc(pb), *as = malloc(sa), *bs = malloc(sb);
  uint8_t *ap_g = malloc(pa), *as_g = malloc(sa);
  float *ref = malloc(sizeof(float) * mn), *cf = malloc(sizeof(float) * mn);
  uint16_t *cb = malloc(2 * mn), *cn = malloc(2 * mn);
  if (!xa || !xb || !ap || !bp || !as || !bs || !ap_g || !as_g || !ref || !cf || !cb || !cn) return 1;
  fill_normal(xa, (size_t)M * K, 1.0f, 1000u + (uint64_t)M);
  fill_normal(xb, (size_t)N * K, 0.02f, 2000u + (uint64_t)N);
  if (mxfp6o_quantise(xa, M, K, fmt_a, ap, as) || mxfp6o_quantise(xb, N, K, fmt_b, bp, bs)) return 1;
  if (mxfp6o_gemm_f32(ap, bp, as, bs, ref, M, N, K, fmt_a, fmt_b)) return 1;

  void *d_xa, *d_ap, *d_bp, *d_as, *d_bs, *d_cf, *d_cb, *d_cn;
  HIP_OK(hipMalloc(&d_xa, sizeof(float) * (size_t)M * K));
  HIP_OK(hipMalloc(&d_ap, pa));
  HIP_OK(hipMalloc(&d_bp, pb));
  HIP_OK(hipMalloc(&d_as, sa));
  HIP_OK(hipMalloc(&d_bs, sb));
  HIP_OK(hipMalloc(&d_cf, sizeof(float) * mn));
  HIP_OK(hipMalloc(&d_cb, 2 * mn));
  HIP_OK(hipMalloc(&d_cn, 2 * mn));
  HIP_OK(hipMemcpy(d_xa, xa, sizeof(float) * (size_t)M * K, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_bp, bp, pb, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_bs, bs, sb, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(d_cf, 0xff, sizeof(float) * mn));
  HIP_OK(hipMemset(d_cb, 0xff, 2 * mn));
  HIP_OK(hipMemset(d_cn, 0xff, 2 * mn));
  HIP_OK(hipDeviceSynchronize());

  /* A is quantised on the GPU, B comes from the host: both producers feed the same operator */
  LIB_OK(mxfp6_quantize((const float *)d_xa, d_ap, d_as, M, K, fmt_a, stream));
  LIB_OK(mxfp6_gemm_f32out(d_ap, d_bp, d_as, d_bs, (float *)d_cf, M, N, K, fmt_a, fmt_b, stream));
  LIB_OK(mxfp6_gemm(d_ap, d_bp, d_as, d_bs, d_cb, M, N, K, fmt_a, fmt_b, stream));
  LIB_OK(mxfp6_gemm_noalloc(d_ap, d_bp, d_as, d_bs, d_cn, M, N, K, fmt_a, fmt_b, 0, stream));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(ap_g, d_ap, pa, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(as_g, d_as, sa, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(cf, d_cf, sizeof(float) * mn, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(cb, d_cb, 2 * mn, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(cn, d_cn, 2 * mn, hipMemcpyDeviceToHost));

  int bad = 0;
  if (memcmp(ap_g, ap, pa) || memcmp(as_g, as, sa)) bad++, printf("  quantiser: GPU bytes differ from the oracle's\n");
  double max_err = 0.0, max_ref = 0.0;
  for (size_t i = 0; i < mn; i++) {
    if (!isfinite(cf[i])) { max_err = INFINITY; break; }
    const double e = fabs((double)cf[i] - (double)ref[i]), r = fabs((double)ref[i]);
    if (e > max_err) max_err = e;
    if (r > max_ref) max_ref = r;
  }
  const double metric = max_ref > 0 ? max_err / max_ref : max_err;  /* max |got - ref| / max |ref| */
  if (!(metric <= 2e-3)) bad++, printf("  fp32 output: metric %.3e exceeds 2e-3\n", metric);
  size_t wrong_bf16 = 0, wrong_noalloc = 0;
  for (size_t i = 0; i < mn; i++) {
    wrong_bf16 += cb[i] != mxfp6o_f32_to_bf16(cf[i]);
    /* bit-identical where both entry points take the same kernel; where mxfp6_gemm takes one the no-allocation path has not,
       the same products are added in another order: within one bf16 step of the fp32 result */
    if (cn[i] != cb[i]) {
      const uint32_t u = (uint32_t)cn[i] << 16;
      float v;
      memcpy(&v, &u, 4);
      wrong_noalloc += !(fabs((double)v - (double)cf[i]) <= fabs((double)cf[i]) * 0.0078125);
    }
  }
  if (wrong_bf16) bad++, printf("  bf16 output: %zu values are not the rounding of the accumulators\n", wrong_bf16);
  if (wrong_noalloc) bad++, printf("  mxfp6_gemm_noalloc: %zu values are more than one bf16 step from the fp32 result\n", wrong_noalloc);
  printf("case M=%d N=%d K=%d fmt=%d,%d: metric %.2e  %s\n", M, N, K, fmt_a, fmt_b, metric, bad ? "FAIL" : "ok");
  fflush(stdout);

  HIP_OK(hipFree(d_xa)); HIP_OK(hipFree(d_ap)); HIP_OK(hipFree(d_bp)); HIP_OK(hipFree(d_as));
  HIP_OK(hipFree(d_bs)); HIP_OK(hipFree(d_cf)); HIP_OK(hipFree(d_cb)); HIP_OK(hipFree(d_cn));
  free(xa); free(xb); free(ap); free(bp); free(as); free(bs); free(ap_g); free(as_g); free(ref); free(cf); free(cb); free(cn);
  return bad;
}

int main(void) {
  if (mxfp6_abi_version() / 100 != MXFP6_ABI_VERSION / 100) {
    fprintf(stderr, "library ABI %d does not match the header's %d\n", mxfp6_abi_version(), MXFP6_ABI_VERSION);
    return 102;
  }
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  if (ndev < 1) { fprintf(stderr, "no GPU\n"); return 103; }
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  /* cfg0's shape, a decode shape (skinny kernel), a few hundred rows (block kernel), ragged edges (generic kernel),
   * a size that takes the re-layout pre-pass and the tiled kernel, and a mixed-format one */
  static const int cases[][5] = {{256, 256, 256, 2, 2}, {16, 2048, 4096, 2, 2}, {384, 1024, 2048, 2, 2}, {37, 100, 96, 3, 2},
                                 {1024, 2048, 1024, 2, 2}, {512, 512, 1024, 3, 2}};
  int bad = 0;
  for (size_t i = 0; i < sizeof(cases) / sizeof(cases[0]); i++) {
    printf("run M=%d N=%d K=%d\n", cases[i][0], cases[i][1], cases[i][2]);
    fflush(stdout);
    bad += run_case(cases[i][0], cases[i][1], cases[i][2], cases[i][3], cases[i][4], stream);
  }
  LIB_OK(mxfp6_release_workspaces());
  HIP_OK(hipStreamDestroy(stream));
  puts(bad ? "SOME FAILED" : "ALL OK");
  return bad;
}
