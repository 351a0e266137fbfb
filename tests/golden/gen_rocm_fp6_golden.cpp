// Generates tests/golden/fp6_tables.json from ROCm's own host-side fp6 conversions
// (hip/hip_fp6.h, a system library routine independent of this repository's code):
//   * fp6 -> fp32 for all 64 codes of e2m3 and e3m2
//   * fp32 -> fp6 (round-to-nearest-even, saturating) for a fixed list of probe values
// Build + run:  tests/golden/gen_golden.sh
#include <hip/hip_fp6.h>
#include <cstdio>
#include <cmath>
#include <vector>
int main() {
  std::vector<float> probes;
  for (int i = -640; i <= 640; i++) probes.push_back(i / 64.0f);          // dense grid over [-10, 10], step 1/64
  for (int i = 0; i <= 512; i++) probes.push_back(i / 16.0f);             // [0, 32], step 1/16 (e3m2 range + saturation)
  for (float v : {0.03125f, 0.0312f, 0.0313f, 0.09375f, 0.0937f, 0.0938f, 1e-8f, 1e8f, 7.74f, 7.75f, 7.76f, 29.0f, 30.0f, 31.9f})
    { probes.push_back(v); probes.push_back(-v); }
  printf("{\n");
  for (int fmt = 2; fmt <= 3; fmt++) {
    auto interp = fmt == 2 ? __HIP_E2M3 : __HIP_E3M2;
    printf("  \"decode_%s\": [", fmt == 2 ? "e2m3" : "e3m2");
    for (int c = 0; c < 64; c++) {
      float f;
      if (fmt == 2) { __hip_fp6_e2m3 x; x.__x = (__hip_fp6_storage_t)c; f = float(x); }
      else { __hip_fp6_e3m2 x; x.__x = (__hip_fp6_storage_t)c; f = float(x); }
      printf("%s%.9e", c ? ", " : "", f);
    }
    printf("],\n  \"encode_%s\": [", fmt == 2 ? "e2m3" : "e3m2");
    for (size_t i = 0; i < probes.size(); i++)
      printf("%s%d", i ? ", " : "", (int)(__hip_cvt_float_to_fp6(probes[i], interp, hipRoundNearest) & 63));
    printf("],\n");
  }
  printf("  \"probes\": [");
  for (size_t i = 0; i < probes.size(); i++) printf("%s%.9e", i ? ", " : "", probes[i]);
  printf("]\n}\n");
  return 0;
}
