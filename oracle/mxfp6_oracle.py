"""CPU oracle for the MXFP6 block-scaled GEMM path  --  TEST INFRASTRUCTURE, NOT PRODUCT.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module; the shipped operator (hipkittensp_amd) never does.

What it restates.  The reference tree (benenzhu/HipKittensP) holds no FP6 source: its
FP6 GEMM lives on an unmounted branch (kernels/gemm/README.md:6-7), so there is no
reference function to follow line by line.  The numerical contract is therefore the one
written in BASELINE.json (configs[0]: per-32 E8M0 scale = 2^(floor(log2(blockmax)) - 2),
fp6 e2m3 round-to-nearest-even, 4 values per 3 bytes, bf16 output, C = A . B^T) together
with the OCP Microscaling (MX) v1.0 closed forms for e2m3 / e3m2 / E8M0.  The structure
mirrors the reference's CPU oracles for its other GEMMs:
  * triple-loop C = A.B^T host reference      tests/unit/warp/register/tile/mma.cu:44-55
  * operand convention (both K-contiguous)    kernels/gemm/bf16fp32/utils.py:28-37
  * output pre-allocated, bf16                analysis/bf16_gemm/mi325x/kernel_8192.cpp:223-224

How each function is pinned (tests/test_oracle.py):
  decode_table      closed form, exhaustive 64 codes, vs golden table produced by ROCm's own
                    host fp6 conversion (amd_hip_fp6.h; tests/golden/fp6_tables.json)
  e8m0_to_f32       exhaustive 255 values vs ldexp
  quantise_codes    brute-force nearest-value search with ties-to-even on a dense grid incl.
                    every midpoint +-1ulp; saturation; vs ROCm host float->fp6 golden vectors
  block_scales      hand-made blocks (powers of two, just below / above, zero, outlier, denormal)
  pack / unpack     hand-written 12-byte known-answer vector + round-trip
  dequantise/gemm   brute-force triple loop on tiny shapes, fp64; invariants (scale doubling,
                    K-block permutation, operand swap = transpose)
  f32_to_bf16       vs torch .to(bfloat16) on CPU
The choices the absent FP6 branch alone could pin (bit order of the packing, zero-block scale
byte) are frozen by this repo's fixtures; the packing is additionally confirmed by the GPU
(the scaled MFMA consumes exactly this bitstream, tests/test_gpu_parity.py).
"""
from __future__ import annotations

import numpy as np

E2M3 = 2  # same numbering as the MFMA cbsz / blgp format field
E3M2 = 3
BLOCK = 32  # elements per E8M0 scale

_FMT = {
    E2M3: dict(ebits=2, mbits=3, bias=1, emax=2, maxval=7.5),
    E3M2: dict(ebits=3, mbits=2, bias=3, emax=4, maxval=28.0),
}


def fmt_info(fmt: int) -> dict:
    if fmt not in _FMT:
        raise ValueError(f"fmt must be 2 (e2m3) or 3 (e3m2), got {fmt}")
    return _FMT[fmt]


def decode_table(fmt: int) -> np.ndarray:
    """64-entry fp6 -> fp32 table (OCP MX v1.0: sign | exponent | mantissa, no inf/NaN)."""
    f = fmt_info(fmt)
    out = np.zeros(64, dtype=np.float32)
    for c in range(64):
        s = (c >> 5) & 1
        e = (c >> f["mbits"]) & ((1 << f["ebits"]) - 1)
        m = c & ((1 << f["mbits"]) - 1)
        if e == 0:  # subnormal: m / 2^mbits * 2^(1 - bias)
            v = (m / (1 << f["mbits"])) * 2.0 ** (1 - f["bias"])
        else:
            v = (1.0 + m / (1 << f["mbits"])) * 2.0 ** (e - f["bias"])
        out[c] = -v if s else v
    return out


def e8m0_to_f32(b) -> np.ndarray:
    """E8M0 byte -> 2^(b-127) as fp32 (b = 255 is NaN in OCP MX; b = 0 is 2^-127, an fp32 subnormal)."""
    b = np.asarray(b, dtype=np.uint8)
    out = np.ldexp(np.float64(1.0), np.minimum(b, 254).astype(np.int32) - 127).astype(np.float32)
    return np.where(b == 255, np.float32(np.nan), out).astype(np.float32)


def block_scales(x: np.ndarray, fmt: int) -> np.ndarray:
    """Per-32 E8M0 byte: biased(floor(log2(blockmax)) - emax), clamped to [0, 254].

    BASELINE.json configs[0]: scale = 2^(floor(log2(blockmax)) - 2) for e2m3 (emax = 2); the
    e3m2 analogue subtracts its emax = 4.  An all-zero block takes biased exponent 0.
    """
    f = fmt_info(fmt)
    x = np.asarray(x, dtype=np.float32)
    rows, K = x.shape
    if K % BLOCK:
        raise ValueError("K must be a multiple of 32")
    amax = np.abs(x.reshape(rows, K // BLOCK, BLOCK)).max(axis=2)
    _, ex = np.frexp(amax)  # amax = m * 2^ex, m in [0.5, 1)  ->  floor(log2) = ex - 1
    e = ex.astype(np.int32) - 1 - f["emax"] + 127
    e = np.where(amax == 0, 0, e)
    return np.clip(e, 0, 254).astype(np.uint8)


def quantise_codes(y: np.ndarray, fmt: int) -> np.ndarray:
    """fp32 (already divided by the block scale) -> fp6 code, round-to-nearest-even, saturating."""
    f = fmt_info(fmt)
    mb, bias = f["mbits"], f["bias"]
    y = np.asarray(y, dtype=np.float32)
    sign = np.signbit(y)
    a = np.abs(y).astype(np.float64)
    a = np.minimum(a, f["maxval"])  # saturate (also maps +inf)
    _, ex = np.frexp(a)
    e = np.maximum(ex.astype(np.int64) - 1, 1 - bias)  # exponent of the binade (subnormals share emin)
    q = np.rint(np.ldexp(a, mb - e))  # rint = ties-to-even; q in [0, 2^(mb+1)]
    v = np.ldexp(q, e - mb)  # the rounded magnitude (exact)
    v = np.minimum(v, f["maxval"])
    # encode magnitude v
    _, ex2 = np.frexp(v)
    e2 = ex2.astype(np.int64) - 1
    normal = v >= 2.0 ** (1 - bias)
    ebits = np.where(normal, e2 + bias, 0)
    mant = np.where(normal, np.ldexp(v, mb - e2) - (1 << mb), np.ldexp(v, mb - (1 - bias)))
    code = (ebits.astype(np.int64) << mb) | mant.astype(np.int64)
    code = np.where(np.isnan(y), (1 << 5) - 1, code)  # NaN input: saturate to max magnitude
    code = code | (sign.astype(np.int64) << 5)
    return code.astype(np.uint8)


def quantise(x: np.ndarray, fmt: int):
    """fp32 [rows, K] -> (codes uint8 [rows, K] in 0..63, scales uint8 [rows, K/32])."""
    x = np.asarray(x, dtype=np.float32)
    rows, K = x.shape
    sc = block_scales(x, fmt)
    # division by a power of two is exact apart from underflow to fp32 subnormals -> do it in fp64
    y = np.ldexp(x.astype(np.float64).reshape(rows, K // BLOCK, BLOCK), (127 - sc.astype(np.int32))[:, :, None])
    codes = quantise_codes(y.reshape(rows, K).astype(np.float64).astype(np.float32), fmt)
    return codes, sc


def pack_fp6(codes: np.ndarray) -> np.ndarray:
    """codes [rows, K] (K % 4 == 0) -> bytes [rows, 3K/4]; value j occupies bits [6j, 6j+6) of the
    row's little-endian bitstream (4 values per 3 bytes; a 32-block is 24 contiguous bytes)."""
    c = np.asarray(codes, dtype=np.uint32)
    rows, K = c.shape
    if K % 4:
        raise ValueError("K must be a multiple of 4")
    c = c.reshape(rows, K // 4, 4) & 63
    w = c[:, :, 0] | (c[:, :, 1] << 6) | (c[:, :, 2] << 12) | (c[:, :, 3] << 18)
    out = np.empty((rows, K // 4, 3), dtype=np.uint8)
    out[:, :, 0] = w & 255
    out[:, :, 1] = (w >> 8) & 255
    out[:, :, 2] = (w >> 16) & 255
    return out.reshape(rows, 3 * K // 4)


def unpack_fp6(packed: np.ndarray) -> np.ndarray:
    p = np.asarray(packed, dtype=np.uint8)
    rows, nb = p.shape
    if nb % 3:
        raise ValueError("packed width must be a multiple of 3")
    p = p.reshape(rows, nb // 3, 3).astype(np.uint32)
    w = p[:, :, 0] | (p[:, :, 1] << 8) | (p[:, :, 2] << 16)
    out = np.empty((rows, nb // 3, 4), dtype=np.uint8)
    for j in range(4):
        out[:, :, j] = (w >> (6 * j)) & 63
    return out.reshape(rows, nb // 3 * 4)


def tile_operand(packed: np.ndarray) -> np.ndarray:
    """Row-major packed [rows, 3K/4] -> tile-major bytes (same shape): tiles of 32 rows x 96 bytes, tile
    (rt, kt) at ((rt * K/128) + kt) * 3072; inside, 16-byte piece c of row r at (r*6 + (c ^ ((r>>3)&1))) * 16.
    Defines the layout of include/mxfp6_gemm.h (MXFP6_LAYOUT_TILE) independently of the GPU converter."""
    p = np.asarray(packed, dtype=np.uint8)
    rows, w = p.shape
    if rows % 32 or w % 96:
        raise ValueError("rows % 32 == 0 and K % 128 == 0 required")
    nkt = w // 96
    x = p.reshape(rows // 32, 32, nkt, 6, 16)                      # [rt, r, kt, c, byte]
    out = np.empty((rows // 32, nkt, 32, 6, 16), dtype=np.uint8)     # [rt, kt, r, slot, byte]
    for r in range(32):
        sw = (r >> 3) & 1
        for c in range(6):
            out[:, :, r, c ^ sw, :] = x[:, r, :, c, :]
    return out.reshape(rows, w)


def tile_scales(scales: np.ndarray) -> np.ndarray:
    """Row-major scales [rows, K/32] -> tile-major [rows, nk4 * 16] (nk4 = ceil(K/512)): the 16 bytes a row has
    for four K-tiles stay together, the 32 rows of a row-tile are adjacent: chunk (rt, g) of 512 bytes at
    ((rt * nk4) + g) * 512, row r at (r % 32) * 16 inside it; K-blocks past K are zero.  Defines the scale half of
    MXFP6_LAYOUT_TILE (include/mxfp6_gemm.h) independently of the GPU converter."""
    s = np.asarray(scales, dtype=np.uint8)
    rows, nkb = s.shape
    if rows % 32 or nkb % 4:
        raise ValueError("rows % 32 == 0 and K % 128 == 0 required")
    nk4 = (nkb + 15) // 16
    padded = np.zeros((rows, nk4 * 16), dtype=np.uint8)
    padded[:, :nkb] = s
    x = padded.reshape(rows // 32, 32, nk4, 16)           # [rt, r, g, byte]
    return np.ascontiguousarray(x.transpose(0, 2, 1, 3)).reshape(rows, nk4 * 16)


def dequantise(packed: np.ndarray, scales: np.ndarray, fmt: int, dtype=np.float32) -> np.ndarray:
    """packed [rows, 3K/4] + scales [rows, K/32] -> values [rows, K] = table[code] * 2^(scale-127).
    Exact in fp32 whenever the result is a normal fp32 number."""
    codes = unpack_fp6(packed)
    rows, K = codes.shape
    v = decode_table(fmt).astype(np.float64)[codes]
    s = np.ldexp(1.0, np.asarray(scales, dtype=np.int32) - 127)
    v = (v.reshape(rows, K // BLOCK, BLOCK) * s[:, :, None]).reshape(rows, K)
    return v.astype(dtype)


def gemm_ref(a_packed, b_packed, a_scale, b_scale, fmt_a=E2M3, fmt_b=E2M3, acc=np.float32) -> np.ndarray:
    """Dequantise-and-matmul: C[M,N] = dq(A)[M,K] . dq(B)[N,K]^T, accumulated in `acc` (fp32 = the
    contract; fp64 = the error yardstick)."""
    A = dequantise(a_packed, a_scale, fmt_a, dtype=acc)
    B = dequantise(b_packed, b_scale, fmt_b, dtype=acc)
    return A @ B.T


def epilogue_ref(acc, bias=None, row_scale=None, col_scale=None, activation=None) -> np.ndarray:
    """The fused epilogue in float64: act(acc * row_scale[:, None] * col_scale[None, :] + bias[None, :]).
    relu = max(y, 0); gelu = 0.5 y (1 + erf(y / sqrt 2)); silu = y / (1 + exp(-y)) -- the textbook forms
    (torch.nn.functional.relu / gelu(approximate="none") / silu).  The reference has no fused epilogue for this
    path (its kernels store the accumulator tile as it is, analysis/bf16_gemm/mi325x/kernel_8192.cpp:223-224), so
    these definitions are pinned by closed forms only: tests/test_oracle.py checks them at points with known values
    and against their defining identities."""
    from scipy.special import erf

    y = np.asarray(acc, dtype=np.float64).copy()
    if row_scale is not None:
        y *= np.asarray(row_scale, dtype=np.float64)[:, None]
    if col_scale is not None:
        y *= np.asarray(col_scale, dtype=np.float64)[None, :]
    if bias is not None:
        y += np.asarray(bias, dtype=np.float64)[None, :]
    if activation in (None, "none"):
        return y
    if activation == "relu":
        return np.maximum(y, 0.0)
    if activation == "gelu":
        return 0.5 * y * (1.0 + erf(y / np.sqrt(2.0)))
    if activation == "silu":
        return y / (1.0 + np.exp(-y))
    raise ValueError(f"unknown activation {activation!r}")


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit pattern (uint16), round-to-nearest-even; NaN stays NaN."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(np.asarray(x, dtype=np.float32))
    return np.where(nan, np.uint16(0x7FC0), r).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """The parity metric: max |got - ref| / max(|ref|, 0.01 * rms(ref)).

    An element-wise relative error is undefined where the exact result cancels to ~0, so the
    denominator is floored at 1 % of the result's RMS.  The bar is 2e-3 (BASELINE.json)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    den = np.maximum(np.abs(ref), max(0.01 * rms, 1e-300))
    return float(np.max(np.abs(got - ref) / den)) if ref.size else 0.0


# ----------------------------------------------------------------------------- workloads
def make_source(kind: str, shape, rng: np.random.Generator) -> np.ndarray:
    """Synthetic fp32 sources named by BASELINE.json's configs."""
    if kind == "normal":  # N(0,1)
        return rng.standard_normal(shape, dtype=np.float32)
    if kind == "weights":  # N(0, 0.02)
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)).astype(np.float32)
    if kind == "weights_outliers":  # N(0,0.02), 1 % of entries multiplied by 8
        w = rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)
        mask = rng.random(shape, dtype=np.float32) < 0.01
        return np.where(mask, w * np.float32(8.0), w).astype(np.float32)
    if kind == "laplace":  # Laplace(0,1), heavy tailed
        return rng.laplace(0.0, 1.0, shape).astype(np.float32)
    raise ValueError(kind)


def make_operand(kind: str, rows: int, K: int, fmt: int, seed: int):
    x = make_source(kind, (rows, K), np.random.default_rng(seed))
    codes, sc = quantise(x, fmt)
    return pack_fp6(codes), sc
