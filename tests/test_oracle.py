"""Pins the CPU oracle (numpy and plain-C restatements) against closed forms, brute force, ROCm's own
host fp6 conversions (tests/golden/fp6_tables.json) and hand-written known answers.  No GPU."""
import json
import math
import os

import numpy as np
import pytest

from oracle import c_oracle as co
from oracle import mxfp6_oracle as o

FMTS = [o.E2M3, o.E3M2]
NAME = {o.E2M3: "e2m3", o.E3M2: "e3m2"}


@pytest.fixture(scope="module")
def golden(golden_dir):
    with open(os.path.join(golden_dir, "fp6_tables.json")) as f:
        return json.load(f)


# ------------------------------------------------------------------ decode
def test_decode_closed_form_values():
    # OCP MX v1.0 table 3/4 landmarks, written by hand
    t2, t3 = o.decode_table(o.E2M3), o.decode_table(o.E3M2)
    assert t2[0b000001] == 0.125 and t2[0b000111] == 0.875          # subnormals m/8
    assert t2[0b001000] == 1.0 and t2[0b011111] == 7.5              # min normal, max
    assert t2[0b111111] == -7.5 and t2[0b100000] == 0.0 and math.copysign(1, t2[0b100000]) == -1
    assert t3[0b000001] == 0.0625 and t3[0b000011] == 0.1875        # subnormals m/4 * 2^-2
    assert t3[0b000100] == 0.25 and t3[0b011111] == 28.0
    assert t3[0b001100] == 1.0 and t3[0b111111] == -28.0


@pytest.mark.parametrize("fmt", FMTS)
def test_decode_matches_rocm_host_library(fmt, golden):
    ref = np.array(golden[f"decode_{NAME[fmt]}"], dtype=np.float32)
    for tab in (o.decode_table(fmt), co.decode_table(fmt)):
        assert tab.dtype == np.float32
        assert np.array_equal(tab.view(np.uint32), ref.view(np.uint32))  # bit-exact, incl. -0


@pytest.mark.parametrize("fmt", FMTS)
def test_decode_monotone_and_symmetric(fmt):
    t = o.decode_table(fmt)
    assert np.all(np.diff(t[:32]) > 0)
    assert np.array_equal(t[32:], -t[:32])


def test_e8m0_exhaustive():
    b = np.arange(255, dtype=np.uint8)
    got = o.e8m0_to_f32(b)
    for i in range(255):
        assert got[i] == math.ldexp(1.0, i - 127)
        assert co.lib().mxfp6o_e8m0(i) == math.ldexp(1.0, i - 127)
    assert np.isnan(o.e8m0_to_f32(np.uint8(255)))
    assert math.isnan(co.lib().mxfp6o_e8m0(255))


# ------------------------------------------------------------------ quantise (element)
def _brute_force_code(y, fmt):
    """nearest representable value, ties to even mantissa code, saturating; independent of the fast path."""
    tab = o.decode_table(fmt).astype(np.float64)[:32]
    a = min(abs(float(y)), 2.0 * tab[-1])  # keep the distance search exact for huge inputs
    d = np.abs(tab - a)
    m = d.min()
    cands = np.nonzero(d == m)[0]
    c = int(cands[0]) if len(cands) == 1 else int([k for k in cands if k % 2 == 0][0])
    return c | (32 if math.copysign(1.0, y) < 0 else 0)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantise_codes_vs_brute_force(fmt):
    tab = o.decode_table(fmt)[:32].astype(np.float64)
    pts = []
    mids = (tab[:-1] + tab[1:]) / 2
    for v in np.concatenate([tab, mids]):
        f = np.float32(v)
        pts += [f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf))]
    pts += [np.float32(x) for x in (tab[-1] * 1.01, tab[-1] * 1.5, 100.0, 1e30, 1e-30, 0.0)]
    pts = np.array(pts + [-p for p in pts], dtype=np.float32)
    rng = np.random.default_rng(7)
    pts = np.concatenate([pts, (rng.standard_normal(4000) * tab[-1] / 2).astype(np.float32)])
    got = o.quantise_codes(pts, fmt)
    exp = np.array([_brute_force_code(p, fmt) for p in pts], dtype=np.uint8)
    assert np.array_equal(got, exp)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantise_codes_vs_rocm_host_library(fmt, golden):
    probes = np.array(golden["probes"], dtype=np.float32)
    exp = np.array(golden[f"encode_{NAME[fmt]}"], dtype=np.uint8)
    got = o.quantise_codes(probes, fmt)
    # ROCm's conversion and ours may differ only in the sign bit of results that round to zero
    same = got == exp
    zero = (got & 31) == 0
    assert np.all(same | (zero & ((got & 31) == (exp & 31))))
    assert np.mean(same) > 0.99


@pytest.mark.parametrize("fmt", FMTS)
def test_saturation_not_wraparound(fmt):
    mx = o.fmt_info(fmt)["maxval"]
    y = np.array([mx, mx * 1.0001, mx * 1.06, mx * 2, np.inf, -mx * 3, -np.inf], dtype=np.float32)
    c = o.quantise_codes(y, fmt)
    assert list(c) == [31, 31, 31, 31, 31, 63, 63]


# ------------------------------------------------------------------ block scale
@pytest.mark.parametrize("fmt", FMTS)
def test_block_scale_rule(fmt):
    emax = o.fmt_info(fmt)["emax"]
    def sc(vals):
        x = np.zeros((1, 32), np.float32); x[0, : len(vals)] = vals
        a, b = o.block_scales(x, fmt)[0, 0], co.quantise(x, fmt)[1][0, 0]
        assert a == b
        return int(a)
    assert sc([1.0]) == 127 - emax                     # floor(log2 1) = 0
    assert sc([1.9999]) == 127 - emax
    assert sc([2.0]) == 128 - emax
    assert sc([-4.0, 0.5]) == 129 - emax               # max of |.|
    assert sc([np.nextafter(np.float32(1), np.float32(0))]) == 126 - emax
    assert sc([0.0]) == 0                              # all-zero block
    assert sc([1e-45]) == 0                            # denormal fp32: clamps at biased 0
    assert sc([3e38]) == min(254, 127 + 127 - emax)
    assert sc([0.02, 0.16]) == 127 - 3 - emax          # one x8 outlier sets the block scale: log2(.16) = -2.64


def test_cfg0_scale_formula_literal():
    # BASELINE.json configs[0]: scale = 2^(floor(log2(blockmax)) - 2) for e2m3
    rng = np.random.default_rng(0)
    x = rng.standard_normal((64, 256), dtype=np.float32)
    sc = o.block_scales(x, o.E2M3)
    bm = np.abs(x.reshape(64, 8, 32)).max(axis=2).astype(np.float64)
    assert np.array_equal(o.e8m0_to_f32(sc).astype(np.float64), 2.0 ** (np.floor(np.log2(bm)) - 2))
    # consequence: |x/scale| < 8 always, so codes saturate only through rounding 7.75.. -> 7.5
    y = x.reshape(64, 8, 32) / o.e8m0_to_f32(sc)[:, :, None]
    assert np.abs(y).max() < 8.0


# ------------------------------------------------------------------ packing
def test_pack_known_answer():
    # codes 0..7 -> bitstream, LSB first: 000000 100000 010000 110000 | ...
    codes = np.array([[1, 2, 3, 4, 63, 0, 32, 21]], dtype=np.uint8)
    # group0: 1 | 2<<6 | 3<<12 | 4<<18 = 0x103081 -> bytes 81 30 10 ; group1: 63 | 0 | 32<<12 | 21<<18 = 0x56003F -> 3F 00 56
    assert o.pack_fp6(codes).tobytes() == bytes([0x81, 0x30, 0x10, 0x3F, 0x00, 0x56])
    assert np.array_equal(o.unpack_fp6(o.pack_fp6(codes)), codes)


def test_pack_roundtrip_and_bit_positions():
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 64, size=(5, 128), dtype=np.uint8)
    p = o.pack_fp6(codes)
    assert p.shape == (5, 96)
    assert np.array_equal(o.unpack_fp6(p), codes)
    bits = np.unpackbits(p, axis=1, bitorder="little")            # value j at bits [6j, 6j+6)
    for j in (0, 1, 5, 31, 32, 127):
        v = sum(int(bits[2, 6 * j + q]) << q for q in range(6))
        assert v == codes[2, j]


def test_tile_major_layout_definition():
    # hand-checked placements: 64 rows, K = 256 (2 K-tiles): piece c of row r, K-tile kt
    p = np.zeros((64, 192), np.uint8)
    def piece(r, kt, c):
        return p[r, kt * 96 + c * 16 : kt * 96 + c * 16 + 16]
    piece(0, 0, 0)[:] = 1      # row 0: no swap -> slot 0 of tile (0,0): byte 0
    piece(0, 1, 5)[:] = 2      # K-tile 1 -> tile (0,1) at 3072; slot 5 -> 3072 + 80
    piece(9, 0, 2)[:] = 3      # row 9 has bit 3 set: piece 2 <-> slot 3 -> (9*6+3)*16 = 912
    piece(40, 1, 1)[:] = 4     # row 40 = row-tile 1 row 8 (bit 3 set): tile (1,1) at (1*2+1)*3072 = 9216; slot 0 -> 9216 + 8*96
    t = o.tile_operand(p).reshape(-1)
    assert t[0] == 1 and t[3072 + 80] == 2 and t[912] == 3 and t[9216 + 768] == 4
    assert int(t.astype(np.int64).sum()) == 16 * (1 + 2 + 3 + 4)
    rng = np.random.default_rng(1)
    q = rng.integers(0, 256, size=(96, 384), dtype=np.uint8)
    tq = o.tile_operand(q)
    assert sorted(tq.reshape(-1).tolist()) == sorted(q.reshape(-1).tolist())


def test_tile_major_scale_layout_definition():
    # hand-checked placements: 64 rows, K = 1152 (36 K-blocks -> nk4 = 3 chunks per row-tile, last one a quarter full)
    s = np.zeros((64, 36), np.uint8)
    s[0, 0] = 1       # row-tile 0, chunk 0, row 0, byte 0 -> 0
    s[5, 17] = 2      # chunk 1 (blocks 16..31), row 5, byte 1 -> 512 + 5*16 + 1
    s[40, 35] = 3     # row-tile 1 (chunks 3..5), chunk 2, row 8, byte 3 -> (3 + 2)*512 + 8*16 + 3
    t = o.tile_scales(s)
    assert t.shape == (64, 48)
    f = t.reshape(-1)
    assert f[0] == 1 and f[512 + 81] == 2 and f[5 * 512 + 131] == 3 and int(f.astype(np.int64).sum()) == 6
    rng = np.random.default_rng(2)
    q = rng.integers(1, 256, size=(96, 32), dtype=np.uint8)   # K = 1024: a pure permutation
    tq = o.tile_scales(q)
    assert tq.shape == q.shape and sorted(tq.reshape(-1).tolist()) == sorted(q.reshape(-1).tolist())
    # the 16 bytes of one row and one group of four K-tiles stay contiguous
    assert np.array_equal(tq.reshape(-1)[(1 * 2 + 1) * 512 + 7 * 16:(1 * 2 + 1) * 512 + 8 * 16], q[39, 16:32])


# ------------------------------------------------------------------ numpy vs C, end to end
@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("kind", ["normal", "weights_outliers", "laplace"])
def test_numpy_and_c_quantisers_bit_identical(fmt, kind):
    x = o.make_source(kind, (37, 256), np.random.default_rng(11))
    x[3, :32] = 0.0
    x[4, 5] = 1e-42
    codes, sc = o.quantise(x, fmt)
    pc, scc = co.quantise(x, fmt)
    assert np.array_equal(sc, scc)
    assert np.array_equal(o.pack_fp6(codes), pc)
    d1, d2 = o.dequantise(pc, scc, fmt), co.dequantise(pc, scc, fmt)
    assert np.array_equal(d1.view(np.uint32), d2.view(np.uint32))
    assert np.array_equal(co.dequantise(pc, scc, fmt, transpose=True), d2.T)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantisation_error_bound(fmt):
    # within a block, |x - dq(q(x))| <= half a step of the top binade unless saturated
    x = o.make_source("normal", (16, 512), np.random.default_rng(5))
    codes, sc = o.quantise(x, fmt)
    d = o.dequantise(o.pack_fp6(codes), sc, fmt)
    f = o.fmt_info(fmt)
    step = o.e8m0_to_f32(sc)[:, :, None] * 2.0 ** (f["emax"] - f["mbits"])
    err = np.abs(d - x).reshape(16, 16, 32)
    sat = np.abs(x).reshape(16, 16, 32) > o.e8m0_to_f32(sc)[:, :, None] * f["maxval"]
    assert np.all((err <= step / 2) | sat)


def test_cfg0_fixture_is_reproducible():
    ap, asc = o.make_operand("normal", 256, 256, o.E2M3, seed=0)
    ap2, asc2 = co.quantise(o.make_source("normal", (256, 256), np.random.default_rng(0)), o.E2M3)
    assert np.array_equal(ap, ap2) and np.array_equal(asc, asc2)
    assert ap.shape == (256, 192) and asc.shape == (256, 8)


# ------------------------------------------------------------------ gemm
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2), (2, 3), (3, 3)])
@pytest.mark.parametrize("M,N,K", [(1, 1, 32), (3, 5, 64), (16, 16, 32), (33, 17, 96), (64, 64, 256)])
def test_gemm_vs_brute_force(fa, fb, M, N, K):
    ap, asc = o.make_operand("normal", M, K, fa, seed=M * 7 + K)
    bp, bsc = o.make_operand("weights_outliers", N, K, fb, seed=N * 13 + K)
    ref = co.gemm_f64_naive(ap, bp, asc, bsc, fa, fb)                 # element-by-element triple loop
    # independent restatement of the same sum in python ints/floats for the smallest case
    if M * N * K <= 3 * 5 * 64:
        ca, cb = o.unpack_fp6(ap), o.unpack_fp6(bp)
        ta, tb = o.decode_table(fa), o.decode_table(fb)
        for i in range(M):
            for j in range(N):
                s = sum(float(ta[ca[i, k]]) * 2.0 ** (int(asc[i, k // 32]) - 127) * float(tb[cb[j, k]]) * 2.0 ** (int(bsc[j, k // 32]) - 127) for k in range(K))
                assert s == pytest.approx(ref[i, j], rel=1e-12, abs=1e-300)
    for got in (o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float32), co.gemm_f32(ap, bp, asc, bsc, fa, fb)):
        assert o.rel_err(got, ref) < 1e-5
    assert o.rel_err(o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64), ref) < 1e-12


def test_gemm_invariants():
    M, N, K = 24, 40, 256
    ap, asc = o.make_operand("laplace", M, K, o.E3M2, seed=1)
    bp, bsc = o.make_operand("weights", N, K, o.E2M3, seed=2)
    C = co.gemm_f32(ap, bp, asc, bsc, 3, 2)
    # +1 on every A scale doubles C exactly
    assert np.array_equal(co.gemm_f32(ap, bp, asc + 1, bsc, 3, 2), 2 * C)
    # operand swap transposes (same accumulation order per element -> exact)
    Ct = co.gemm_f32(bp, ap, bsc, asc, 2, 3)
    assert o.rel_err(Ct.T, C) < 1e-5
    # permuting whole K-blocks (with their scales) in both operands leaves the exact result unchanged
    perm = np.random.default_rng(0).permutation(K // 32)
    def pk(p, s):
        return p.reshape(-1, K // 32, 24)[:, perm].reshape(p.shape), s[:, perm]
    ap2, asc2 = pk(ap, asc); bp2, bsc2 = pk(bp, bsc)
    assert np.allclose(co.gemm_f64_naive(ap2, bp2, asc2, bsc2, 3, 2), co.gemm_f64_naive(ap, bp, asc, bsc, 3, 2), rtol=1e-12, atol=1e-300)
    # a block whose codes are all zero contributes nothing whatever its scale
    ap3 = ap.copy(); ap3.reshape(M, K // 32, 24)[:, 0] = 0
    asc3 = asc.copy(); asc3[:, 0] = 254
    ap4 = ap3.copy(); asc4 = asc.copy(); asc4[:, 0] = 0
    assert np.array_equal(co.gemm_f32(ap3, bp, asc3, bsc, 3, 2), co.gemm_f32(ap4, bp, asc4, bsc, 3, 2))
    # one-hot B (code 1.0, scale 127) reads back dequantised A: the decode is bit exact through the gemm
    eye_codes = np.zeros((K, K), np.uint8); eye_codes[np.arange(K), np.arange(K)] = 0b001000
    ep, esc = o.pack_fp6(eye_codes), np.full((K, K // 32), 127, np.uint8)
    assert np.array_equal(co.gemm_f32(ap, ep, asc, esc, 3, 2), o.dequantise(ap, asc, 3))


def test_cfg0_end_to_end_cpu():
    """BASELINE.json configs[0]: 256^3 e2m3, N(0,1) seed 0 (A) / seed 1 (B), bf16 output."""
    ap, asc = o.make_operand("normal", 256, 256, o.E2M3, seed=0)
    bp, bsc = o.make_operand("normal", 256, 256, o.E2M3, seed=1)
    ref64 = o.gemm_ref(ap, bp, asc, bsc, acc=np.float64)
    c32 = co.gemm_f32(ap, bp, asc, bsc)
    assert o.rel_err(c32, ref64) < 2e-3
    bits = co.gemm_bf16_bits(ap, bp, asc, bsc)
    assert np.array_equal(bits, o.f32_to_bf16_bits(c32))
    # and the quantised product is a sane approximation of the unquantised one
    xa = o.make_source("normal", (256, 256), np.random.default_rng(0)).astype(np.float64)
    xb = o.make_source("normal", (256, 256), np.random.default_rng(1)).astype(np.float64)
    exact = xa @ xb.T
    assert np.sqrt(np.mean((ref64 - exact) ** 2)) / np.sqrt(np.mean(exact ** 2)) < 0.06


def test_bf16_rounding_vs_torch():
    import torch
    rng = np.random.default_rng(9)
    x = np.concatenate([rng.standard_normal(10000).astype(np.float32) * 100,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf, 1e-40], np.float32)])
    exp = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(o.f32_to_bf16_bits(x), exp)
    got_c = np.array([co.lib().mxfp6o_f32_to_bf16(float(v)) for v in x[-200:]], dtype=np.uint16)
    assert np.array_equal(got_c, exp[-200:])
    assert np.array_equal(o.bf16_bits_to_f32(exp).view(np.uint32) >> 16, exp.astype(np.uint32))


def test_epilogue_closed_forms():
    """The fused-epilogue definitions at points with known values and through their identities (a wrong sign,
    a dropped 1/2 or sqrt 2, scale and bias applied in the wrong order or along the wrong axis all fail here)."""
    y = np.array([[-3.0, -1.0, 0.0, 0.5, 2.0]])
    assert np.array_equal(o.epilogue_ref(y, activation="relu"), [[0.0, 0.0, 0.0, 0.5, 2.0]])
    g = o.epilogue_ref(y, activation="gelu")
    # Phi(1) = 0.841344746068543, Phi(2) = 0.977249868051821, Phi(3) = 0.998650101968370 (standard normal CDF)
    assert np.allclose(g, [[-3 * (1 - 0.998650101968370), -(1 - 0.841344746068543), 0.0, 0.5 * 0.691462461274013, 2 * 0.977249868051821]], atol=1e-14)
    assert np.allclose(g - o.epilogue_ref(-y, activation="gelu"), y, atol=1e-14)        # gelu(y) - gelu(-y) = y
    s = o.epilogue_ref(y, activation="silu")
    assert np.allclose(s, y / (1 + np.exp(-y))) and np.allclose(s - o.epilogue_ref(-y, activation="silu"), y)  # silu(y) - silu(-y) = y
    assert np.isclose(s[0, 4], 2 / (1 + np.exp(-2.0))) and np.isclose(s[0, 1], -0.2689414213699951)
    acc = np.arange(6, dtype=np.float64).reshape(2, 3)
    out = o.epilogue_ref(acc, bias=[10, 20, 30], row_scale=[1, 2], col_scale=[1, 10, 100])
    assert np.array_equal(out, [[10, 30, 230], [16, 100, 1030]])  # (acc * rs * cs) + bias, bias per column, rs per row
