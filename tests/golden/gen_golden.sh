#!/bin/sh
# Regenerates tests/golden/fp6_tables.json from ROCm's host fp6 conversions (needs hipcc; no GPU).
set -e
cd "$(dirname "$0")"
hipcc -x hip --offload-arch=gfx950 -o /tmp/gen_rocm_fp6_golden gen_rocm_fp6_golden.cpp
/tmp/gen_rocm_fp6_golden > fp6_tables.json
