"""Builds hipkittensp_amd/libmxfp6_gemm.so (gfx950 only) from csrc/*.hip with hipcc, and libmxfp6_probes.so beside it.

    python -m hipkittensp_amd.build            # rebuild everything
The libraries are built in-tree; nothing is installed.  No GPU is needed to build.

libmxfp6_gemm.so is the operator (include/mxfp6_gemm.h).  libmxfp6_probes.so is the measurement build
(include/mxfp6_probes.h): the same objects, except that the C ABI and the e2m3 x e2m3 instantiations of the LDS-tiled
kernel are compiled a second time with -DMXFP6_PROBES (probe entry points, ablation builds, clock stamps) and the probe
kernels (csrc/probes.hip) are added.  bench.py loads it for its ceilings and ablations; the operator never does.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmxfp6_gemm.so")
PROBES_LIB = os.path.join(HERE, "libmxfp6_probes.so")
SOURCES = ["api.hip", "dispatch.hip", "gemm_generic.hip", "gemm_tiled.hip", "gemm_tiled4.hip", "gemm_block.hip", "gemm_mid.hip", "gemm_skinny.hip", "gemm_ring.hip", "quantize.hip"]
# (source, object name, extra flags).  gemm_tiled.hip gives five objects: its host-side part, and the kernel
# instantiations of each pair of operand formats (the bulk of the build time; they compile side by side).
UNITS = [(src, src.replace(".hip", ""), []) for src in SOURCES] + [
    ("gemm_tiled.hip", f"gemm_tiled_fmt{fmt}", [f"-DMXFP6_TILED_FMT={fmt}"]) for fmt in (22, 23, 32, 33)
]
# what the measurement build compiles again (or in addition), with -DMXFP6_PROBES
PROBE_UNITS = [("api.hip", "api_probes", ["-DMXFP6_PROBES"]), ("gemm_tiled.hip", "gemm_tiled_fmt22_probes", ["-DMXFP6_TILED_FMT=22", "-DMXFP6_PROBES"]),
               ("probes.hip", "probes", ["-DMXFP6_PROBES"])]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-std=c++20", "-O3", "-fPIC", "-fvisibility=hidden",
    # packed-fp32 VALU forms are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile(unit) -> str:
    src, name, extra = unit
    obj = os.path.join(OBJ, name + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on {src} ({name}):\n{err}")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    # the units that take longest first
    order = sorted(UNITS + PROBE_UNITS, key=lambda u: (u[1] != "gemm_block", not u[1].startswith("gemm_tiled_fmt"), u[1] not in ("gemm_skinny", "gemm_mid")))
    with cf.ThreadPoolExecutor(max_workers=min(8, len(order))) as ex:
        objs = dict(zip((u[1] for u in order), ex.map(_compile, order)))
    product = [objs[u[1]] for u in UNITS]
    swapped = {"api": "api_probes", "gemm_tiled_fmt22": "gemm_tiled_fmt22_probes"}
    probes = [objs[swapped.get(u[1], u[1])] for u in UNITS] + [objs["probes"]]
    for lib, members in ((LIB, product), (PROBES_LIB, probes)):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *members]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            raise RuntimeError(f"link failed:\n{r.stderr}")
        if verbose:
            print(f"built {lib}")
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
