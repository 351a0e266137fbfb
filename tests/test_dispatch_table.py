"""The kernel choice's calibration table and time model, without a GPU: the committed table is what the committed sweep
gives under the model as built (so nobody changes the model's constants and ships a table made for the old ones), and the
model's figures behave as a time should."""
import ctypes
import json
import os

import pytest

from hipkittensp_amd import _lib, calibrate

CANDIDATES = ["tiled_256x256", "tiled_128x256", "tiled_128x128", "block", "block_128x256", "skinny", "tiled_k_split_256", "tiled_k_split_128", "block_k_split", "ring"]


@pytest.fixture(scope="module")
def model():
    P = _lib.probes()
    P.mxfp6_probe_candidate.restype = ctypes.c_int
    P.mxfp6_probe_candidate.argtypes = [ctypes.c_int] * 6 + [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int)]

    def f(M, N, K, layouts, cand, cus=256):
        m, c, sh = ctypes.c_double(), ctypes.c_double(), ctypes.c_int()
        rc = P.mxfp6_probe_candidate(M, N, K, layouts, CANDIDATES.index(cand), cus, ctypes.byref(m), ctypes.byref(c), ctypes.byref(sh))
        assert rc == 0, rc
        return m.value, c.value, sh.value

    return f


def test_committed_table_belongs_to_the_committed_sweep_and_the_built_model(tmp_path):
    sweep = json.load(open(calibrate.SWEEP))
    assert sweep["candidates"] == CANDIDATES
    out = tmp_path / "table.inc"
    n = calibrate.write_table(sweep, str(out))
    assert n == len(sweep["points"]) > 1000
    assert out.read_text() == open(calibrate.TABLE).read(), "run `python -m hipkittensp_amd.calibrate hipkittensp_amd/csrc/dispatch_sweep.json` and rebuild"


def test_table_is_sorted_into_buckets():
    rows, buckets = [], []
    section = None
    for line in open(calibrate.TABLE):
        if "kCalPoints[]" in line:
            section = rows
        elif "kCalBuckets[]" in line:
            section = buckets
        elif line.startswith("  {") and section is not None:
            section.append([int(x.strip(" {}")) for x in line.strip().split(",")[:4]])
    assert len(rows) > 1000 and sum(b[3] for b in buckets) == len(rows)
    keys = [(r[3], r[0]) for r in rows]          # (layouts, M)
    assert keys == sorted(keys)
    for layouts, M, first, count in buckets:
        assert all(k == (layouts, M) for k in keys[first:first + count])
        assert first == 0 or keys[first - 1] != (layouts, M)


def test_model_figures_behave_like_times(model):
    # applicability: the skinny kernel up to 128 rows, the ring kernel up to 256, a split only where the tiles leave CUs idle
    assert model(16, 8192, 28672, 0, "skinny")[0] > 0 and model(256, 8192, 28672, 0, "skinny")[0] < 0
    assert model(256, 8192, 28672, 2, "ring")[0] > 0 and model(512, 8192, 28672, 2, "ring")[0] < 0
    assert model(8192, 8192, 8192, 3, "tiled_k_split_256")[0] < 0 and model(256, 8192, 28672, 3, "tiled_k_split_256")[2] == 8
    assert model(128, 8192, 28672, 3, "block_k_split")[2] > 1
    # more work takes longer; tile-major operands are never slower in the model; half the CUs never make a large GEMM faster
    for cand in ("tiled_256x256", "block", "tiled_128x256"):
        t1, t2 = model(4096, 4096, 4096, 3, cand)[0], model(4096, 4096, 8192, 3, cand)[0]
        assert 0 < t1 < t2 < 2.2 * t1
        assert model(4096, 4096, 4096, 3, cand)[0] <= model(4096, 4096, 4096, 0, cand)[0]
        assert model(8192, 8192, 8192, 3, cand, cus=128)[0] > model(8192, 8192, 8192, 3, cand, cus=256)[0]
    # 8192^3 on the tiled kernel: the model knows the chip's sustained rate (3.5 - 4.2 PFLOP/s)
    t = model(8192, 8192, 8192, 3, "tiled_256x256")[0]
    assert 2 * 8192 ** 3 / 4.2e15 * 1e6 < t < 2 * 8192 ** 3 / 3.3e15 * 1e6
    # at a calibrated shape the calibrated figure is the measured one (to the table's three decimals and the blend with neighbours)
    sweep = json.load(open(calibrate.SWEEP))
    p = next(q for q in sweep["points"] if (q["M"], q["N"], q["K"], q["layouts"]) == (512, 8192, 8192, 3))
    cal = model(512, 8192, 8192, 3, "block")[1]
    assert abs(cal / p["measured_us"][CANDIDATES.index("block")] - 1) < 0.05
