"""GPU parity: the HIP path (called through the C ABI via hipkittensp_amd.tk_kernel) against the CPU
oracle on the same seeded inputs.  Bars (BASELINE.json): fp6 -> fp32 decode bit-exact; GEMM within
max relative error 2e-3 of the dequantise-and-matmul result, measured on the fp32 accumulators
before the bf16 rounding (metric: oracle.rel_err); bf16 output = RNE of those accumulators;
quantiser bit-exact.  Full-size configurations are checked on sampled rows/columns against the
fp64 oracle plus size-independent properties (exact scale linearity, operand swap = transpose,
kernel-vs-kernel agreement)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import mxfp6_oracle as o

pytestmark = pytest.mark.gpu

TOL = 2e-3  # BASELINE.json north_star: max relative error vs the fp32 dequantise-and-matmul
# What the hardware actually delivers, measured on MI355X: with at least one e2m3 operand every fp6
# product and every partial sum of these workloads is exactly representable and the scaled MFMA
# returns the fp64 result rounded once (metric 0 .. 1e-7), so those cases are held to 1e-5.  With
# e3m2 on BOTH operands the MFMA's internal sum of the 64 products of a K-pair is itself inexact
# (|err| up to 3e-5 of sum|a||b|, metric up to 6e-3 where results cancel); that combination is not
# one of BASELINE.json's configurations and is held to 1e-2 plus a bound relative to sum|a||b|.
TOL_TIGHT = 1e-5
TOL_E3M2_BOTH = 1e-2


def tol(fa, fb):
    return TOL_E3M2_BOTH if (fa == 3 and fb == 3) else TOL_TIGHT


def check(got, ref, fa, fb, ap=None, asc=None, bp=None, bsc=None):
    assert np.isfinite(got).all()
    e = o.rel_err(got, ref)
    assert e <= tol(fa, fb), f"rel_err {e} > {tol(fa, fb)} for formats {fa},{fb}"
    if fa == 3 and fb == 3 and ap is not None:
        l1 = np.abs(o.dequantise(ap, asc, fa, np.float64)) @ np.abs(o.dequantise(bp, bsc, fb, np.float64)).T
        assert np.max(np.abs(got - ref) / np.maximum(l1, 1e-300)) <= 1e-4


@pytest.fixture(scope="module")
def hk():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import hipkittensp_amd as m
    from hipkittensp_amd import _lib

    _lib.lib()  # fails loudly if the HIP library is not built: there is no fallback path
    prev = m.tk_kernel.allow_e3m2_pair(True)   # the tests of that pair know its bound (TOL_E3M2_BOTH); test_e3m2_pair_needs_opt_in checks the default
    yield m
    m.tk_kernel.allow_e3m2_pair(prev)
    m.tk_kernel.set_kernel(0)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def gemm(hk, ap, bp, asc, bsc, fa=2, fb=2, out="f32", kernel=0):
    M, N = ap.shape[0], bp.shape[0]
    C = torch.full((M, N), float("nan"), dtype=torch.float32 if out == "f32" else torch.bfloat16, device="cuda")
    prev = hk.tk_kernel.set_kernel(kernel)
    try:
        hk.dispatch_micro(dev(ap), dev(bp), dev(asc), dev(bsc), C, fa, fb)
        torch.cuda.synchronize()
    finally:
        hk.tk_kernel.set_kernel(prev)
    if out == "f32":
        return C.cpu().numpy()
    return C.view(torch.int16).cpu().numpy().view(np.uint16)


def gemm_probes_lib(ap, bp, asc, bsc, fa=2, fb=2, kernel=0):
    """The same call through the measurement build of the library (libmxfp6_probes.so), whose overrides (raster, clock
    stamps, ablations) only its own entry points see; fp32 output."""
    from hipkittensp_amd import _lib

    P = _lib.probes()
    M, N, K = ap.shape[0], bp.shape[0], ap.shape[1] // 3 * 4
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    dA, dB, dAs, dBs = dev(ap), dev(bp), dev(asc), dev(bsc)
    prev = P.mxfp6_set_kernel(kernel)
    try:
        rc = P.mxfp6_gemm_ex(dA.data_ptr(), dB.data_ptr(), dAs.data_ptr(), dBs.data_ptr(), C.data_ptr(), M, N, K, fa, fb, 0, 0, 1, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
    finally:
        P.mxfp6_set_kernel(prev)
    return C.cpu().numpy()


def operands(M, N, K, fa, fb, seed, kind_a="normal", kind_b="normal"):
    xa = o.make_source(kind_a, (M, K), np.random.default_rng(seed))
    xb = o.make_source(kind_b, (N, K), np.random.default_rng(seed + 1000))
    ap, asc = co.quantise(xa, fa)
    bp, bsc = co.quantise(xb, fb)
    return ap, asc, bp, bsc


def one_hot_b(K):
    codes = np.zeros((K, K), np.uint8)
    codes[np.arange(K), np.arange(K)] = 0b001000  # 1.0 in e2m3
    return o.pack_fp6(codes), np.full((K, K // 32), 127, np.uint8)


def test_e3m2_pair_needs_opt_in(hk):
    """e3m2 x e3m2 can exceed the 2e-3 bar (the MFMA's own sum of such products is inexact): by default the operator
    refuses the pair with a distinct error, and runs it once the caller has accepted the weaker bound."""
    ap, asc, bp, bsc = operands(64, 64, 256, 3, 3, seed=5)
    prev = hk.tk_kernel.allow_e3m2_pair(False)
    try:
        with pytest.raises(RuntimeError, match="e3m2 x e3m2"):
            gemm(hk, ap, bp, asc, bsc, 3, 3)
        gemm(hk, ap, bp, asc, bsc, 3, 2)   # every other pair runs
        assert hk.tk_kernel.allow_e3m2_pair(True) is False
        check(gemm(hk, ap, bp, asc, bsc, 3, 3), o.gemm_ref(ap, bp, asc, bsc, 3, 3, acc=np.float64), 3, 3, ap, asc, bp, bsc)
    finally:
        hk.tk_kernel.allow_e3m2_pair(prev)


# ------------------------------------------------------------------ decode: bit exact
@pytest.mark.parametrize("kernel,M", [(1, 64), (1, 37), (2, 256), (3, 16), (3, 32), (3, 5)])
@pytest.mark.parametrize("fmt", [2, 3])
def test_decode_bit_exact_through_the_mfma(hk, kernel, M, fmt):
    K = 512 if kernel == 3 else 256
    rng = np.random.default_rng(fmt * 10 + kernel)
    codes = rng.integers(0, 64, size=(M, K), dtype=np.uint8)
    codes[0, :64] = np.arange(64)  # every code of the format at least once
    ap = o.pack_fp6(codes)
    asc = rng.integers(110, 140, size=(M, K // 32), dtype=np.uint8)
    bp, bsc = one_hot_b(K)
    got = gemm(hk, ap, bp, asc, bsc, fmt, 2, kernel=kernel)
    exp = o.dequantise(ap, asc, fmt)
    # bit for bit, except that the code -0 comes back as +0: an accumulator that starts at +0 cannot return -0
    nz = exp != 0
    assert np.array_equal(got.view(np.uint32)[nz], exp.view(np.uint32)[nz])
    assert np.all(got[~nz] == 0)


# ------------------------------------------------------------------ BASELINE configs[0]
@pytest.mark.parametrize("kernel", [0, 1, 2])
def test_cfg0_256_cubed(hk, kernel):
    ap, asc = o.make_operand("normal", 256, 256, 2, seed=0)
    bp, bsc = o.make_operand("normal", 256, 256, 2, seed=1)
    ref64 = o.gemm_ref(ap, bp, asc, bsc, acc=np.float64)
    c32 = gemm(hk, ap, bp, asc, bsc, kernel=kernel)
    assert o.rel_err(c32, ref64) <= TOL_TIGHT <= TOL
    assert o.rel_err(c32, co.gemm_f32(ap, bp, asc, bsc)) <= TOL           # vs the fp32 CPU path itself
    cb = gemm(hk, ap, bp, asc, bsc, out="bf16", kernel=kernel)
    assert np.array_equal(cb, o.f32_to_bf16_bits(c32))                     # epilogue = RNE of the accumulators
    assert o.rel_err(o.bf16_bits_to_f32(cb), ref64) <= 2.0 ** -8 + TOL


# ------------------------------------------------------------------ generic kernel: ragged shapes
@pytest.mark.parametrize("M,N,K", [(1, 1, 32), (5, 3, 64), (31, 33, 96), (32, 32, 32), (65, 127, 160), (100, 40, 1024), (257, 255, 416)])
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2), (2, 3), (3, 3)])
def test_generic_kernel_any_shape(hk, M, N, K, fa, fb):
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M + N + K, kind_b="weights_outliers")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=1)
    check(got, ref, fa, fb, ap, asc, bp, bsc)
    cb = gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=1)
    assert np.array_equal(cb, o.f32_to_bf16_bits(got))


# ------------------------------------------------------------------ tiled kernel
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (256, 512, 384), (512, 256, 1664), (768, 1024, 1024),
                                   (300, 264, 256), (257, 8, 128), (100, 1000, 384), (33, 520, 640), (1, 256, 128)])  # edge tiles too
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2), (2, 3), (3, 3)])
@pytest.mark.parametrize("kernel", [2, 18])  # 8-wave ping-pong (the one the automatic choice uses) and the 4-wave interleaved schedule
def test_tiled_kernel_vs_oracle(hk, M, N, K, fa, fb, kernel):
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M * 3 + N + K, kind_a="laplace" if fa == 3 else "normal", kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel)
    check(got, ref, fa, fb, ap, asc, bp, bsc)
    cb = gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=kernel)
    assert np.array_equal(cb, o.f32_to_bf16_bits(got))


# ------------------------------------------------------------------ ring kernel (batched decode: private streams of B, flag-guarded ring of A)
@pytest.mark.parametrize("M,N,K", [(1, 128, 512), (16, 256, 2048), (17, 1000, 1024), (32, 132, 3584), (33, 520, 2048), (64, 4096, 4096), (64, 8192, 8192),
                                   (100, 264, 1536), (128, 384, 8192), (129, 132, 1024), (200, 520, 28672), (256, 1024, 4096), (300, 4, 512)])
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2), (2, 3), (3, 3)])
def test_ring_kernel_vs_oracle(hk, M, N, K, fa, fb):
    """One, two and four row-tiles of A per workgroup, several blocks of rows, ragged M and N, every K split the shape allows
    (shares 1, the automatic number, 3): against the fp64 oracle; bf16 output = RNE of the fp32 output; the sum over the
    shares is taken in share order whoever arrives last, so a call repeated gives the same bits."""
    tk = hk.tk_kernel
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M * 7 + N + K, kind_a="laplace" if fa == 3 else "normal", kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    for shares in (1, 0, 3):
        prev = tk.set_k_split(shares)
        try:
            got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=tk.KERNEL_RING)
            check(got, ref, fa, fb, ap, asc, bp, bsc)
            assert np.array_equal(gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=tk.KERNEL_RING), o.f32_to_bf16_bits(got))
            assert np.array_equal(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=tk.KERNEL_RING), got)
        finally:
            tk.set_k_split(prev)


def test_ring_kernel_rejects_what_it_cannot_take(hk):
    tk = hk.tk_kernel
    for M, N, K in ((64, 128, 640), (64, 130, 1024), (64, 128, 256)):   # K % 512 != 0, N % 4 != 0, K < 512
        ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=3)
        with pytest.raises(RuntimeError):
            gemm(hk, ap, bp, asc, bsc, kernel=tk.KERNEL_RING)


# ------------------------------------------------------------------ block kernel (128 x 128 tiles, four waves in step)
@pytest.mark.parametrize("M,N,K", [(128, 128, 512), (256, 384, 1024), (512, 256, 2560), (300, 264, 1536), (129, 8, 512), (100, 1000, 1024), (33, 520, 2048),
                                   (1, 128, 512), (640, 1024, 4096), (256, 256, 128), (300, 264, 640), (100, 520, 1152), (257, 8, 384)])  # edge tiles too; K % 512 != 0: a last group of fewer than four K-tiles
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2), (2, 3), (3, 3)])
@pytest.mark.parametrize("kernel", [23, 24, 26])  # ring of three slots (two workgroups per CU), of six (one); tiles of 128 x 256
def test_block_kernel_vs_oracle(hk, M, N, K, fa, fb, kernel):
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M * 5 + N + K, kind_a="laplace" if fa == 3 else "normal", kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel)
    check(got, ref, fa, fb, ap, asc, bp, bsc)
    cb = gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=kernel)
    assert np.array_equal(cb, o.f32_to_bf16_bits(got))
    assert np.array_equal(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=22), got)   # ring depth chosen by the library, 128 x 128 tiles: same bits


@pytest.mark.parametrize("M,N,K,la,lb", [(256, 8192, 2048, 1, 1), (192, 4096, 4096, 0, 1), (512, 3072, 3072, 0, 0), (1024, 2048, 8192, 1, 1), (96, 16384, 1024, 0, 1),
                                         (384, 6144, 4096, 1, 0), (2048, 4096, 1024, 1, 1),   # 512 tiles, two workgroups per CU
                                         (640, 12808, 640, 0, 0), (24, 12032, 768, 0, 0)])    # a very short K against a row-major B: 505 tiles with a ragged last column; few rows
def test_block_kernel_matches_the_tiled_kernel(hk, M, N, K, la, lb):
    """Shapes of the kind the block kernel is for (its tiles do not outnumber the CUs, K of moderate length): whatever the
    automatic path takes without a K split, the forced block kernel and the 8-wave tiled kernel give the same bits (same
    order of summation along K), and the result passes against the fp64 oracle on sampled rows."""
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=M + N + K, kind_b="weights")
    A, As = (hk.tile_operand(dev(ap)), hk.tile_scales(dev(asc), K)) if la else (dev(ap), dev(asc))
    B, Bs = (hk.tile_operand(dev(bp)), hk.tile_scales(dev(bsc), K)) if lb else (dev(bp), dev(bsc))
    outs = {}
    for kernel in (0, 22, 2):
        C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        prev, prev_split = hk.tk_kernel.set_kernel(kernel), hk.tk_kernel.set_k_split(1)
        try:
            hk.dispatch_micro(A, B, As, Bs, C, layout_a=la, layout_b=lb)
            torch.cuda.synchronize()
        finally:
            hk.tk_kernel.set_kernel(prev)
            hk.tk_kernel.set_k_split(prev_split)
        outs[kernel] = C.cpu().numpy()
    assert np.array_equal(outs[0], outs[22]) and np.array_equal(outs[22], outs[2])
    rows = np.random.default_rng(M).choice(M, 16, replace=False)
    check(outs[22][rows], o.gemm_ref(ap[rows], bp, asc[rows], bsc, acc=np.float64), 2, 2)


@pytest.mark.parametrize("M,N,K,shares", [(128, 256, 4096, 2), (128, 512, 8192, 4), (100, 264, 4096, 2), (256, 512, 8192, 8), (64, 1024, 16384, 0), (192, 2048, 8192, 0),
                                          (128, 256, 32768, 16), (200, 136, 18432, 9),   # many shares
                                          (128, 512, 8192, 0), (96, 520, 28672, 0), (100, 128, 16384, 0), (512, 512, 28672, 0),
                                          # K % 512 != 0: the last share takes what is left of K, down to a single K-tile
                                          (128, 256, 2816, 2), (100, 264, 4480, 3), (128, 384, 4224, 4), (16, 4096, 11008, 0), (256, 512, 11008, 0), (64, 1024, 18944, 0)])
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2)])
def test_block_kernel_k_split(hk, M, N, K, shares, fa, fb):
    """The block kernel with the K range of every output tile split between several workgroups: fp32 partial matrices in
    the stream's workspace, summed in share order by the tiled kernel's reduction.  Forced share counts on the forced
    kernel, and shapes on which the automatic path may choose this split itself.  Against the fp64 oracle; bf16 output = RNE
    of the fp32 output; a second call gives the same bits; tile-major operands give the same bits as row-major ones; a
    fused epilogue is applied by the reduction."""
    tk = hk.tk_kernel
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M + N + K + shares, kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    kernel = 22 if shares else 0
    prev = tk.set_k_split(shares)
    try:
        got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel)
        check(got, ref, fa, fb, ap, asc, bp, bsc)
        assert np.array_equal(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel), got)
        assert np.array_equal(gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=kernel), o.f32_to_bf16_bits(got))
        if N % 32 == 0:
            C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            pk = tk.set_kernel(kernel)
            try:
                hk.dispatch_micro(dev(ap), hk.tile_operand(dev(bp)), dev(asc), hk.tile_scales(dev(bsc), K), C, fa, fb, layout_b=1)
                torch.cuda.synchronize()
            finally:
                tk.set_kernel(pk)
            if shares:
                assert np.array_equal(C.cpu().numpy(), got)
            else:
                check(C.cpu().numpy(), ref, fa, fb, ap, asc, bp, bsc)  # the automatic path may take another split for another layout
        bias = torch.linspace(-1, 1, N, device="cuda")
        C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        pk = tk.set_kernel(kernel)
        try:
            hk.dispatch_micro(dev(ap), dev(bp), dev(asc), dev(bsc), C, fa, fb, bias=bias, activation="relu")
            torch.cuda.synchronize()
        finally:
            tk.set_kernel(pk)
        want = np.maximum(got + bias.cpu().numpy()[None, :], 0)
        assert np.allclose(C.cpu().numpy(), want, rtol=1e-6, atol=1e-6 * np.abs(got).max())
    finally:
        tk.set_k_split(prev)


# The automatic choice is judged by what it costs, not by which kernel it names: on this list of shapes (decode and batched
# decode against row-major and tile-major weights, a few hundred rows, prefill-sized and square problems, a K no K split
# divides, wide and narrow N) the call as the library dispatches it must be within 10 % of the fastest forced candidate.
CHOICE_SHAPES = [(16, 8192, 28672, 0, 0), (16, 8192, 28672, 0, 1), (32, 8192, 28672, 0, 1), (64, 8192, 28672, 0, 1), (64, 8192, 28672, 0, 0),
                 (128, 8192, 28672, 0, 1), (256, 8192, 28672, 1, 1), (512, 8192, 8192, 1, 1), (256, 8192, 8192, 0, 1), (1024, 8192, 8192, 0, 1),
                 (64, 28672, 8192, 0, 0), (32, 28672, 4096, 0, 1), (128, 4096, 14336, 0, 1), (2048, 4096, 4096, 1, 1), (96, 10240, 8192, 0, 1),
                 (16, 4096, 11008, 0, 1), (4096, 4096, 4096, 0, 0), (48, 57344, 8192, 0, 0), (192, 2048, 8192, 0, 1), (8, 2048, 8192, 0, 0)]


def test_automatic_choice_is_within_ten_percent_of_the_best_forced_candidate(hk):
    """Timed as the calibration is: on the GPU's side (mxfp6_probe_time_gemm of the measurement build, back-to-back launches
    between two events) with the weights rotating through about 400 MB, so that they come from HBM."""
    import ctypes

    from hipkittensp_amd import _lib

    tk, P = hk.tk_kernel, _lib.probes()
    candidates = ((tk.KERNEL_TILED, 1), (tk.KERNEL_TILED_128, 1), (tk.KERNEL_TILED_256, 1), (tk.KERNEL_TILED_128x128, 1), (tk.KERNEL_BLOCK, 1), (tk.KERNEL_BLOCK_WIDE, 1),
                  (tk.KERNEL_SKINNY, 0), (tk.KERNEL_MID, 0), (tk.KERNEL_RING, 0), (tk.KERNEL_TILED_256, -1), (tk.KERNEL_TILED_128, -1), (tk.KERNEL_BLOCK, -1))
    g = torch.Generator(device="cuda")
    g.manual_seed(123)
    stream = torch.cuda.current_stream().cuda_stream

    behind = {}
    for M, N, K, la, lb in CHOICE_SHAPES:
        a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2, layout=la)
        b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2, layout=lb)
        sets = min(16, max(2, -(-400_000_000 // (N * K * 3 // 4))))
        B, Bs = torch.stack([b] * sets), torch.stack([bsc] * sets)   # the same weights at `sets` addresses: what matters is where they come from
        C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        us = ctypes.c_double()

        def time_us(kernel, split):
            pk, ps = P.mxfp6_set_kernel(kernel), P.mxfp6_set_k_split(split)
            try:
                rc = P.mxfp6_probe_time_gemm(a.data_ptr(), B.data_ptr(), asc.data_ptr(), Bs.data_ptr(), C.data_ptr(), M, N, K, 2, 2, la, lb, 0, sets,
                                             B.stride(0), Bs.stride(0), 3, 24, ctypes.byref(us), stream)
            finally:
                P.mxfp6_set_kernel(pk)
                P.mxfp6_set_k_split(ps)
            return us.value if rc == 0 else None   # None: the forced kernel does not take the shape

        ratio = None
        for attempt in range(3):   # timings on a shared box scatter: the best of up to three rounds counts
            auto = time_us(tk.KERNEL_AUTO, 0)
            forced = [t for t in (time_us(k, sp) for k, sp in candidates) if t is not None]
            auto = min(auto, time_us(tk.KERNEL_AUTO, 0))
            r = auto / min(forced)
            ratio = r if ratio is None else min(ratio, r)
            if ratio <= 1.10:
                break
        if ratio > 1.10:
            behind[(M, N, K, la, lb)] = round(ratio, 3)
        del B, Bs, C
    assert len(behind) <= 1 and all(r <= 1.25 for r in behind.values()), behind


def test_kernel_choice_reports_the_unambiguous_cases(hk):
    """mxfp6_kernel_choice on shapes where one kernel is the only sensible answer."""
    tk = hk.tk_kernel
    assert tk.kernel_choice(8192, 8192, 8192) == tk.KERNEL_TILED and tk.kernel_choice(8192, 8192, 8192, 1, 1) == tk.KERNEL_TILED
    assert tk.kernel_choice(16, 8192, 28672) in (tk.KERNEL_SKINNY, tk.KERNEL_RING)   # level with each other there
    assert tk.kernel_choice(4, 4096, 4096) == tk.KERNEL_SKINNY
    assert tk.kernel_choice(40, 36, 96) == tk.KERNEL_GENERIC
    assert tk.kernel_choice(64, 8192, 28672, 0, 1) == tk.KERNEL_RING and tk.kernel_choice(64, 28672, 8192, 0, 0) == tk.KERNEL_RING
    assert tk.kernel_choice(512, 8192, 8192, 1, 1) == tk.KERNEL_BLOCK
    assert tk.kernel_choice(128, 512, 16384) in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT) and tk.kernel_choice(256, 8192, 28672, 1, 1) in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT)
    prev = tk.set_k_split(1)   # no K split (the ring kernel may still be taken, as one share)
    try:
        assert tk.kernel_choice(128, 512, 16384) not in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT)
        assert tk.kernel_choice(64, 8192, 28672, 0, 1) not in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT, tk.KERNEL_RING)
    finally:
        tk.set_k_split(prev)


def test_block_kernel_rejects_what_it_cannot_take(hk):
    ap, asc, bp, bsc = operands(128, 128, 96, 2, 2, seed=1)       # K % 128
    with pytest.raises(RuntimeError, match="bad shape"):
        gemm(hk, ap, bp, asc, bsc, kernel=22)
    ap, asc, bp, bsc = operands(128, 36, 512, 2, 2, seed=1)       # N % 8
    with pytest.raises(RuntimeError, match="bad shape"):
        gemm(hk, ap, bp, asc, bsc, kernel=23)


@pytest.mark.parametrize("M,N,K,shares", [(256, 512, 4096, 2), (256, 512, 4096, 4), (300, 264, 8192, 4), (128, 768, 8192, 8), (100, 520, 2048, 2),
                                          (512, 256, 16384, 0), (96, 1024, 14336, 0), (160, 2048, 8192, 0)])
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2)])
def test_tiled_kernel_k_split(hk, M, N, K, shares, fa, fb):
    """The tiled kernel with the K range of every output tile split between several workgroups (few output tiles, long K):
    fp32 partial matrices in the stream's workspace, summed in share order by a second kernel.  Forced share counts on the
    forced tiled kernel, and shapes on which the automatic path chooses the split itself (asserted through the plan probe).
    Against the fp64 oracle; bf16 output = RNE of the fp32 output; a second call gives the same bits; tile-major operands
    give the same bits as row-major ones; the fused epilogue agrees with the unsplit kernel's."""
    tk = hk.tk_kernel
    n, rows = tk.k_split_plan(M, N, K, 0, shares if shares else -1)   # the split these shapes have when they are to split
    assert n > 1 and rows in (128, 256), (n, rows)
    if shares > 1:
        assert n == shares
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M + N + K + shares, kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    kernel = 2   # the tiled kernel forced; shares = 0: its split wherever the shape has one
    prev = tk.set_k_split(shares if shares else -1)
    try:
        got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel)
        check(got, ref, fa, fb, ap, asc, bp, bsc)
        assert np.array_equal(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel), got)
        cb = gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=kernel)
        assert np.array_equal(cb, o.f32_to_bf16_bits(got))
        dA, dB, dAs, dBs = dev(ap), dev(bp), dev(asc), dev(bsc)
        pk = tk.set_kernel(kernel)
        try:
            if M % 32 == 0 and N % 32 == 0:
                C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
                hk.dispatch_micro(hk.tile_operand(dA), hk.tile_operand(dB), hk.tile_scales(dAs, K), hk.tile_scales(dBs, K), C, fa, fb, layout_a=1, layout_b=1)
                assert np.array_equal(C.cpu().numpy(), got)
            rng = np.random.default_rng(M + K)
            bias, rs = dev(rng.standard_normal(N).astype(np.float32)), dev((0.5 + rng.random(M)).astype(np.float32))
            F = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            hk.dispatch_micro(dA, dB, dAs, dBs, F, fa, fb, bias=bias, row_scale=rs, activation="silu")
            tk.set_k_split(1)
            U = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            hk.dispatch_micro(dA, dB, dAs, dBs, U, fa, fb, bias=bias, row_scale=rs, activation="silu")
            assert o.rel_err(F.cpu().numpy(), U.cpu().numpy()) <= 1e-5
        finally:
            tk.set_kernel(pk)
    finally:
        tk.set_k_split(prev)


def test_k_split_plans_are_whole_and_bounded(hk):
    """The mechanical part of a K split (how many shares, once a shape is to split): every share a whole number of groups of
    four K-tiles and at least eight K-tiles, the shares of all tiles on at most the CUs, none where K is no multiple of 512."""
    tk = hk.tk_kernel
    for M, N, K in [(256, 8192, 28672), (128, 4096, 14336), (1024, 1024, 16384), (768, 2048, 8192), (96, 8192, 8192), (512, 256, 16384)]:
        n, rows = tk.k_split_plan(M, N, K, 0, -1)
        tiles = -(-M // rows) * -(-N // 256)
        assert n > 1 and rows in (128, 256) and (K // 512) % n == 0 and K // 128 // n >= 8 and tiles * n <= 256, (M, N, K, n, rows)
    for M, N, K in [(4096, 4096, 16384), (64, 264, 101 * 128), (256, 512, 1024)]:   # more tiles than half the CUs; K % 512 != 0; K too short
        assert tk.k_split_plan(M, N, K, 0, -1)[0] == 1, (M, N, K)
    assert tk.k_split_plan(256, 512, 8192, 0, 1)[0] == 1     # 1 = never


def test_forced_kernels_reject_shapes_they_cannot_take(hk):
    ap, asc, bp, bsc = operands(64, 64, 64, 2, 2, seed=1)
    with pytest.raises(RuntimeError, match="bad shape"):
        gemm(hk, ap, bp, asc, bsc, kernel=2)
    ap, asc, bp, bsc = operands(129, 64, 512, 2, 2, seed=1)
    with pytest.raises(RuntimeError, match="bad shape"):
        gemm(hk, ap, bp, asc, bsc, kernel=3)          # M > 128
    ap, asc, bp, bsc = operands(16, 64, 384, 2, 2, seed=1)
    with pytest.raises(RuntimeError, match="bad shape"):
        gemm(hk, ap, bp, asc, bsc, kernel=3)          # K % 512
    check(gemm(hk, ap, bp, asc, bsc, kernel=0), o.gemm_ref(ap, bp, asc, bsc, acc=np.float64), 2, 2)  # automatic: tiled
    ap, asc, bp, bsc = operands(40, 36, 96, 2, 2, seed=2)
    with pytest.raises(RuntimeError, match="bad shape"):
        gemm(hk, ap, bp, asc, bsc, kernel=2)          # N % 8, K % 128
    check(gemm(hk, ap, bp, asc, bsc, kernel=0), o.gemm_ref(ap, bp, asc, bsc, acc=np.float64), 2, 2)  # automatic: generic


# ------------------------------------------------------------------ automatic path over random shapes
def test_automatic_path_random_shapes_against_the_generic_kernel(hk):
    """Sixty seeded random shapes and layout pairs through the automatic choice, each against the generic kernel (which the
    oracle tests pin) on the same bytes: whatever kernel, tile shape, ring depth or K split the rules pick, the fp32 result
    agrees to the rounding of the sums.  The draw covers every kernel the choice can make."""
    tk = hk.tk_kernel
    rng = np.random.default_rng(2024)
    seen = set()
    for case in range(60):
        kind = case % 6
        if kind == 0:      # few rows, long K
            M, N, K = int(rng.integers(1, 65)), int(rng.integers(1, 65)) * 128, int(rng.integers(4, 57)) * 512
        elif kind == 1:    # a few hundred rows, K of moderate length
            M, N, K = int(rng.integers(65, 769)), int(rng.integers(8, 65)) * 128, int(rng.integers(2, 17)) * 512
        elif kind == 2:    # a few hundred rows, long K, narrow N
            M, N, K = int(rng.integers(33, 513)), int(rng.integers(1, 33)) * 128, int(rng.integers(16, 57)) * 512
        elif kind == 3:    # ragged everything (N % 8 == 0, K % 128 == 0)
            M, N, K = int(rng.integers(1, 700)), int(rng.integers(1, 300)) * 8, int(rng.integers(1, 40)) * 128
        elif kind == 4:    # many tiles
            M, N, K = int(rng.integers(4, 17)) * 128, int(rng.integers(16, 33)) * 128, int(rng.integers(1, 9)) * 512
        else:              # K % 32 only: the generic kernel's own
            M, N, K = int(rng.integers(1, 200)), int(rng.integers(1, 200)), int(rng.integers(1, 30)) * 32
        la = int(rng.integers(0, 2)) if M % 32 == 0 and K % 128 == 0 else 0
        lb = int(rng.integers(0, 2)) if N % 32 == 0 and K % 128 == 0 else 0
        seen.add(tk.kernel_choice(M, N, K, la, lb))
        g = torch.Generator(device="cuda"); g.manual_seed(case)
        a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2, la)
        b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.05, 3 if case % 5 == 0 else 2, lb)
        fb = 3 if case % 5 == 0 else 2
        ref = torch.empty(M, N, dtype=torch.float32, device="cuda")
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ar, asr = (hk.tile_operand(a, untile=True), hk.tile_scales(asc, K, untile=True)) if la else (a, asc)
        br, bsr = (hk.tile_operand(b, untile=True), hk.tile_scales(bsc, K, untile=True)) if lb else (b, bsc)
        prev = tk.set_kernel(1)
        try:
            hk.dispatch_micro(ar, br, asr, bsr, ref, 2, fb)
        finally:
            tk.set_kernel(prev)
        hk.dispatch_micro(a, b, asc, bsc, got, 2, fb, layout_a=la, layout_b=lb)
        torch.cuda.synchronize()
        assert o.rel_err(got.cpu().numpy(), ref.cpu().numpy()) <= TOL_TIGHT, (case, M, N, K, la, lb)
    assert tk.KERNEL_GENERIC in seen and len(seen) >= 4, seen   # the cases spread over the kernel families


# ------------------------------------------------------------------ skinny kernel
@pytest.mark.parametrize("M,N,K", [(16, 64, 512), (1, 32, 1024), (7, 100, 2048), (16, 512, 3584), (32, 96, 1536), (13, 33, 512 * 9), (17, 31, 512 * 13), (16, 1000, 512 * 20),
                                   (33, 40, 1024), (64, 96, 512 * 5), (48, 1000, 2048), (50, 31, 512 * 11),    # 33 - 64 rows of A: two accumulator tiles
                                   (65, 40, 1024), (128, 96, 512 * 5), (100, 1000, 2048), (96, 31, 512 * 11)])  # 65 - 128: four, half chunks
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2)])
def test_skinny_kernel_vs_oracle(hk, M, N, K, fa, fb):
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M + 2 * N + K, kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=3)
    check(got, ref, fa, fb, ap, asc, bp, bsc)
    cb = gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=3)
    assert np.array_equal(cb, o.f32_to_bf16_bits(got))
    # every workgroup geometry (32 rows of B, 16 rows, 32 rows with half the waves) sums the same products; the order of the
    # partial sums differs, so they agree to fp32 rounding, and each is held to the oracle
    for kern in (hk.tk_kernel.KERNEL_SKINNY_32, hk.tk_kernel.KERNEL_SKINNY_16, hk.tk_kernel.KERNEL_SKINNY_HALF):
        check(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kern), ref, fa, fb, ap, asc, bp, bsc)
    # the K range split between 2 / 4 / 8 workgroups per tile of C (more splits than chunks leaves some without work);
    # twice each: the tile counters must be back at zero after a launch
    check(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=hk.tk_kernel.KERNEL_SKINNY_2WAVES), ref, fa, fb, ap, asc, bp, bsc)
    check(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=hk.tk_kernel.KERNEL_SKINNY_64), ref, fa, fb, ap, asc, bp, bsc)  # 64 rows of B per workgroup
    for kern in hk.tk_kernel.KERNEL_SKINNY_32_SPLIT + hk.tk_kernel.KERNEL_SKINNY_16_SPLIT + hk.tk_kernel.KERNEL_SKINNY_64_SPLIT:
        for _ in range(2):
            check(gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kern), ref, fa, fb, ap, asc, bp, bsc)


@pytest.mark.parametrize("kernel", [3, 7, 8, 9, 11, 13, 16, 19, 20])
@pytest.mark.parametrize("M,N,K", [(16, 4096, 4096), (32, 2080, 1536), (5, 17408, 1024), (64, 4096, 2048), (100, 2080, 1536), (128, 17408, 1024), (40, 16416, 8192)])
def test_skinny_geometries_tile_major_weights(hk, kernel, M, N, K):
    """Each geometry with tile-major weights and scales (16 rows per workgroup read half of every 3 KB tile) against the
    generic kernel on the row-major operands; ragged N only row-major."""
    g = torch.Generator(device="cuda"); g.manual_seed(N + K)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2)
    ref = torch.empty(M, N, dtype=torch.float32, device="cuda")
    prev = hk.tk_kernel.set_kernel(1)
    try:
        hk.dispatch_micro(a, b, asc, bsc, ref)
        hk.tk_kernel.set_kernel(kernel)
        for lb in ((0, 1) if N % 32 == 0 else (0,)):
            B, Bs = (hk.tile_operand(b), hk.tile_scales(bsc, K)) if lb else (b, bsc)
            C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            hk.dispatch_micro(a, B, asc, Bs, C, layout_b=lb)
            torch.cuda.synchronize()
            assert o.rel_err(C.cpu().numpy(), ref.cpu().numpy()) <= TOL_TIGHT, (kernel, lb)
    finally:
        hk.tk_kernel.set_kernel(prev)


def test_skinny_k_split_chosen_by_shape_streams_and_capture(hk):
    """Few rows of B and a long K: the automatic choice splits K between workgroups (partial tiles in a per-stream
    workspace, summed by the last workgroup to arrive).  Against the generic kernel; tile-major weights; fused epilogue;
    two streams at once, each with its own workspace; under stream capture (a workspace exists or the launch runs
    unsplit: the same sums up to fp32 rounding either way)."""
    M, N, K = 16, 1024, 28672
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2)
    bias = torch.randn(N, device="cuda", generator=g)
    bt, bst = hk.tile_operand(b), hk.tile_scales(bsc, K)
    ref = torch.empty(M, N, dtype=torch.float32, device="cuda")
    prev = hk.tk_kernel.set_kernel(1)
    try:
        hk.dispatch_micro(a, b, asc, bsc, ref)
    finally:
        hk.tk_kernel.set_kernel(prev)
    torch.cuda.synchronize()
    refn = ref.cpu().numpy()
    for rep in range(3):
        for B, Bs, lb in ((b, bsc, 0), (bt, bst, 1)):
            C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            hk.dispatch_micro(a, B, asc, Bs, C, layout_b=lb)
            assert o.rel_err(C.cpu().numpy(), refn) <= TOL_TIGHT, (rep, lb)
    C = torch.empty(M, N, dtype=torch.float32, device="cuda")
    hk.dispatch_micro(a, bt, asc, bst, C, layout_b=1, bias=bias, activation="relu")
    assert torch.allclose(C, torch.relu(ref + bias[None, :]), rtol=2e-6, atol=1e-5)
    # two streams, launches interleaved
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda") for _ in range(6)] for _ in streams]
    torch.cuda.synchronize()
    for i in range(6):
        for st, out in zip(streams, outs):
            with torch.cuda.stream(st):
                hk.dispatch_micro(a, bt, asc, bst, out[i], layout_b=1)
    torch.cuda.synchronize()
    for out in outs:
        for C in out:
            assert o.rel_err(C.cpu().numpy(), refn) <= TOL_TIGHT
    # capture and replays
    Cg = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hk.dispatch_micro(a, bt, asc, bst, Cg, layout_b=1)
    for rep in range(3):
        Cg.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert o.rel_err(Cg.cpu().numpy(), refn) <= TOL_TIGHT, f"replay {rep}"
        hk.dispatch_micro(a, bt, asc, bst, torch.empty_like(Cg), layout_b=1)
        torch.cuda.synchronize()


@pytest.mark.parametrize("block", [True, False])
def test_k_split_streams_and_capture(hk, block):
    """A K split on a shape where the automatic path chooses one (a few hundred rows of A, long K) -- the block kernel's,
    and with the tiled kernel forced, the tiled kernel's own: against the generic kernel; two streams at once, each
    with its own workspace of partial sums; under stream capture on a stream that has its workspace already (captured
    with the split) and replayed with eager work in between."""
    M, N, K = 192, 1024, 16384
    tk = hk.tk_kernel
    assert tk.kernel_choice(M, N, K) in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT) and tk.k_split_plan(M, N, K, 0, -1)[0] > 1
    prev = tk.set_kernel(tk.KERNEL_AUTO if block else tk.KERNEL_TILED)
    try:
        _k_split_streams_and_capture(hk, M, N, K)
    finally:
        tk.set_kernel(prev)


def test_capture_on_a_stream_without_workspace_runs_unsplit(hk):
    """A shape the automatic path would split, captured on a stream that has never launched one: the library may not
    allocate during capture, so the graph holds the unsplit launch; every replay gives the eager (split) result to
    fp32 rounding of the sums, and nothing is left allocated by the capture."""
    M, N, K = 192, 1024, 16384
    assert hk.tk_kernel.kernel_choice(M, N, K) in (hk.tk_kernel.CHOICE_BLOCK_K_SPLIT, hk.tk_kernel.CHOICE_TILED_K_SPLIT)
    g = torch.Generator(device="cuda"); g.manual_seed(10)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2)
    eager = torch.empty(M, N, dtype=torch.float32, device="cuda")
    hk.dispatch_micro(a, b, asc, bsc, eager)
    torch.cuda.synchronize()
    fresh = torch.cuda.Stream()
    Cg = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    graph = torch.cuda.CUDAGraph()
    fresh.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=fresh):
        hk.dispatch_micro(a, b, asc, bsc, Cg)
    for rep in range(2):
        Cg.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert o.rel_err(Cg.cpu().numpy(), eager.cpu().numpy()) <= TOL_TIGHT, f"replay {rep}"


def _k_split_streams_and_capture(hk, M, N, K):
    g = torch.Generator(device="cuda"); g.manual_seed(9)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2)
    ref = torch.empty(M, N, dtype=torch.float32, device="cuda")
    prev = hk.tk_kernel.set_kernel(1)
    try:
        hk.dispatch_micro(a, b, asc, bsc, ref)
    finally:
        hk.tk_kernel.set_kernel(prev)   # the caller's setting: automatic, or the tiled kernel forced
    torch.cuda.synchronize()
    refn = ref.cpu().numpy()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda") for _ in range(6)] for _ in streams]
    torch.cuda.synchronize()
    for i in range(6):
        for st, out in zip(streams, outs):
            with torch.cuda.stream(st):
                hk.dispatch_micro(a, b, asc, bsc, out[i])
    torch.cuda.synchronize()
    for out in outs:
        for C in out:
            assert o.rel_err(C.cpu().numpy(), refn) <= TOL_TIGHT
    # capture on a stream that has launched the split before (torch's recipe: warm up on the side stream, then capture there)
    side = torch.cuda.Stream()
    Cg = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        hk.dispatch_micro(a, b, asc, bsc, Cg)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = Cg.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        hk.dispatch_micro(a, b, asc, bsc, Cg)
    for rep in range(3):
        Cg.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Cg, eager), f"replay {rep}"
        hk.dispatch_micro(a, b, asc, bsc, torch.empty_like(Cg))
        torch.cuda.synchronize()


# ------------------------------------------------------------------ mid-M kernel
@pytest.mark.parametrize("M,N,K", [(33, 32, 1024), (64, 64, 1024), (48, 100, 2048), (64, 520, 3072), (65, 40, 1024), (128, 96, 4096), (100, 33, 2048),
                                   (200, 72, 1024), (256, 160, 5120), (129, 31, 3072),
                                   (64, 8320, 1024), (40, 8250, 2048), (160, 4200, 1024), (256, 4160, 2048), (500, 2100, 1024)])   # 64 rows of B per workgroup
@pytest.mark.parametrize("fa,fb", [(2, 2), (3, 2), (2, 3)])
def test_mid_kernel_vs_oracle(hk, M, N, K, fa, fb):
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M + 2 * N + K, kind_a="laplace", kind_b="weights_outliers")
    ref = o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64)
    got = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=4)
    check(got, ref, fa, fb, ap, asc, bp, bsc)
    cb = gemm(hk, ap, bp, asc, bsc, fa, fb, out="bf16", kernel=4)
    assert np.array_equal(cb, o.f32_to_bf16_bits(got))


def test_mid_kernel_is_chosen_and_rejects_other_shapes(hk):
    # more than 128 rows of A, few 256x256 tiles, K in whole B slots: the automatic choice is the mid kernel and agrees with
    # the forced one bit for bit; up to 128 rows (and N within one round of workgroups) it is the skinny kernel
    ap, asc, bp, bsc = operands(160, 288, 2048, 2, 2, seed=9, kind_b="weights")
    assert np.array_equal(gemm(hk, ap, bp, asc, bsc, kernel=0), gemm(hk, ap, bp, asc, bsc, kernel=4))
    check(gemm(hk, ap, bp, asc, bsc, kernel=4), o.gemm_ref(ap, bp, asc, bsc, acc=np.float64), 2, 2)
    ap, asc, bp, bsc = operands(96, 288, 2048, 2, 2, seed=9, kind_b="weights")
    assert np.array_equal(gemm(hk, ap, bp, asc, bsc, kernel=0), gemm(hk, ap, bp, asc, bsc, kernel=3))
    check(gemm(hk, ap, bp, asc, bsc, kernel=4), o.gemm_ref(ap, bp, asc, bsc, acc=np.float64), 2, 2)
    for M, N, K in ((32, 64, 1024), (520, 64, 1024), (64, 64, 1536)):   # M <= 32, M > 512, K % 1024
        ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=5)
        with pytest.raises(RuntimeError, match="bad shape"):
            gemm(hk, ap, bp, asc, bsc, kernel=4)


# ------------------------------------------------------------------ tile-major operand layout
@pytest.mark.parametrize("rows,K", [(32, 128), (64, 512), (256, 1152), (96, 8192), (64, 640)])
def test_tile_operand_matches_format_definition(hk, rows, K):
    rng = np.random.default_rng(rows + K)
    p = rng.integers(0, 256, size=(rows, K // 4 * 3), dtype=np.uint8)
    t = hk.tile_operand(dev(p))
    torch.cuda.synchronize()
    assert np.array_equal(t.cpu().numpy(), o.tile_operand(p))                       # bit exact vs the CPU definition
    assert np.array_equal(hk.tile_operand(t, untile=True).cpu().numpy(), p)         # and back
    x = o.make_source("normal", (rows, K), rng)
    pt, st = hk.quantize(dev(x), 2, layout=hk.LAYOUT_TILE)                          # quantiser emitting it directly
    pr, sr = co.quantise(x, 2)
    assert np.array_equal(pt.cpu().numpy(), o.tile_operand(pr)) and np.array_equal(st.cpu().numpy(), o.tile_scales(sr))
    ts = hk.tile_scales(dev(sr), K)                                                 # scale converter, both ways
    assert np.array_equal(ts.cpu().numpy(), o.tile_scales(sr))
    assert np.array_equal(hk.tile_scales(ts, K, untile=True).cpu().numpy(), sr)


@pytest.mark.parametrize("kernel,M,N,K", [(23, 256, 512, 1024), (24, 320, 544, 1536), (26, 256, 1024, 1024), (1, 64, 96, 256), (1, 32, 64, 1152), (2, 256, 512, 640), (2, 512, 256, 2048), (2, 288, 96, 384), (2, 320, 544, 1152),
                                          (18, 256, 512, 640), (18, 320, 544, 1152), (3, 16, 128, 1024), (3, 7, 64, 512), (3, 32, 96, 2560), (4, 64, 96, 2048), (4, 160, 64, 1024), (4, 64, 8320, 1024), (4, 192, 4160, 1024), (0, 32, 32, 128), (28, 32, 128, 1024), (28, 64, 544, 4096), (28, 160, 256, 2048)])
@pytest.mark.parametrize("la,lb", [(0, 1), (1, 0), (1, 1)])
def test_tile_major_operands_give_identical_results(hk, kernel, M, N, K, la, lb):
    if kernel in (3, 4) and la == 1:
        pytest.skip("the skinny and mid-M kernels take a row-major A (M need not be a multiple of 32)")
    fa, fb = 3, 2
    ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=M + N + K + la, kind_a="laplace", kind_b="weights")
    if la == 1 and M % 32:
        pytest.skip("tile-major needs rows % 32 == 0")
    ref = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=kernel)
    A = hk.tile_operand(dev(ap)) if la else dev(ap)
    B = hk.tile_operand(dev(bp)) if lb else dev(bp)
    As = hk.tile_scales(dev(asc), K) if la else dev(asc)
    Bs = hk.tile_scales(dev(bsc), K) if lb else dev(bsc)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    prev = hk.tk_kernel.set_kernel(kernel)
    try:
        hk.dispatch_micro(A, B, As, Bs, C, fa, fb, layout_a=la, layout_b=lb)
        torch.cuda.synchronize()
    finally:
        hk.tk_kernel.set_kernel(prev)
    assert np.array_equal(C.cpu().numpy(), ref)      # same kernel, same arithmetic order: bit for bit
    check(ref, o.gemm_ref(ap, bp, asc, bsc, fa, fb, acc=np.float64), fa, fb)


@pytest.mark.parametrize("rows,K,fmt", [(32, 128, 2), (96, 1152, 3), (256, 640, 2), (64, 8192, 2)])
def test_weight_blob_round_trip(hk, rows, K, fmt):
    """The serialised tile-major operand: header as documented, body = the CPU definition of the tile-major layouts
    (oracle.tile_operand / tile_scales) of CPU-generated bytes, unpack = the original, and the views of a blob are usable
    as a tile-major B without conversion."""
    rng = np.random.default_rng(rows + K)
    packed = rng.integers(0, 256, (rows, K // 4 * 3), dtype=np.uint8)
    scales = rng.integers(100, 150, (rows, K // 32), dtype=np.uint8)
    blob = hk.pack_weights(dev(packed), dev(scales), fmt)
    raw = blob.cpu().numpy()
    assert raw[:16].tobytes() == b"MX6T" + bytes([1, fmt, 1, 0]) + rows.to_bytes(4, "little") + K.to_bytes(4, "little")
    nop = rows * (K // 4 * 3)
    assert np.array_equal(raw[16:16 + nop].reshape(rows, -1), o.tile_operand(packed))
    st = o.tile_scales(scales)
    got_s = raw[16 + nop:].reshape(rows, -1)
    assert got_s.shape == st.shape
    valid = o.tile_scales(np.ones_like(scales)) == 1      # the bytes of K-blocks past K are padding (written as 0)
    assert np.array_equal(got_s[valid], st[valid]) and not got_s[~valid].any()
    op, sc, f = hk.unpack_weights(blob)
    assert f == fmt and np.array_equal(hk.tile_operand(op.contiguous(), untile=True).cpu().numpy(), packed)
    assert np.array_equal(hk.tile_scales(sc.contiguous(), K, untile=True).cpu().numpy(), scales)
    # through the C ABI's own unpack as well
    from hipkittensp_amd import _lib
    p2, s2 = torch.empty(rows, K // 4 * 3, dtype=torch.uint8, device="cuda"), torch.empty(rows, K // 32, dtype=torch.uint8, device="cuda")
    assert _lib.lib().mxfp6_blob_unpack(blob.data_ptr(), p2.data_ptr(), s2.data_ptr(), rows, K, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(p2.cpu().numpy(), packed) and np.array_equal(s2.cpu().numpy(), scales)
    # the views are a tile-major B as they are (same result as the row-major operand, bit for bit)
    ap, asc, bp, bsc = operands(48, rows, K, 2, fmt, seed=rows, kind_b="weights")
    blob2 = hk.pack_weights(dev(bp), dev(bsc), fmt)
    B, Bs, _ = hk.unpack_weights(blob2)
    C1 = torch.empty(48, rows, dtype=torch.float32, device="cuda")
    C2 = torch.empty_like(C1)
    hk.dispatch_micro(dev(ap), dev(bp), dev(asc), dev(bsc), C1, 2, fmt)
    hk.dispatch_micro(dev(ap), B, dev(asc), Bs, C2, 2, fmt, layout_b=hk.LAYOUT_TILE)
    torch.cuda.synchronize()
    assert torch.equal(C1, C2)
    corrupt = blob.clone()
    corrupt[4] = 9
    with pytest.raises(RuntimeError, match="blob"):
        hk.unpack_weights(corrupt)


def test_tile_major_rejects_bad_shapes(hk):
    ap, asc, bp, bsc = operands(48, 32, 128, 2, 2, seed=3)
    C = torch.empty(48, 32, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="tile-major"):
        hk.dispatch_micro(dev(ap), dev(bp), dev(asc), dev(bsc), C, layout_a=hk.LAYOUT_TILE)
    with pytest.raises(RuntimeError, match="layout"):
        hk.dispatch_micro(dev(ap), dev(bp), dev(asc), dev(bsc), C, layout_b=7)


def test_cfg1_and_cfg3_tile_major_full_size(hk):
    M = N = K = 8192
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=1)
    dA, dB, dAs, dBs = dev(ap), dev(bp), dev(asc), dev(bsc)
    C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    Ct = torch.empty_like(C)
    hk.dispatch_micro(dA, dB, dAs, dBs, C)
    hk.dispatch_micro(hk.tile_operand(dA), hk.tile_operand(dB), hk.tile_scales(dAs, K), hk.tile_scales(dBs, K), Ct, layout_a=1, layout_b=1)
    assert torch.equal(C, Ct)
    prev = hk.tk_kernel.set_relayout(False)     # the row-major kernel itself, without the re-layout pre-pass of this size
    try:
        assert prev is True
        Ct.zero_()
        hk.dispatch_micro(dA, dB, dAs, dBs, Ct)
        assert torch.equal(C, Ct)
    finally:
        hk.tk_kernel.set_relayout(prev)
    del dA, dB, C, Ct
    M, N, K = 16, 8192, 28672
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=3, kind_b="weights")
    dA, dB, dAs, dBs = dev(ap), dev(bp), dev(asc), dev(bsc)
    C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    Ct = torch.empty_like(C)
    hk.dispatch_micro(dA, dB, dAs, dBs, C)
    hk.dispatch_micro(dA, hk.tile_operand(dB), dAs, hk.tile_scales(dBs, K), Ct, layout_b=1)
    torch.cuda.synchronize()
    assert torch.equal(C, Ct)


# ------------------------------------------------------------------ automatic dispatch over ragged shapes
def test_automatic_dispatch_agrees_with_generic_kernel_on_ragged_shapes(hk):
    """Whatever kernel the library picks (skinny, mid-M, tiled, generic; row- or tile-major operands), the result agrees with
    the independent one-wave-per-tile kernel on the row-major operands.  Seeded; shapes straddle every dispatch boundary."""
    rng = np.random.default_rng(2024)
    ks = [32, 96, 128, 384, 512, 640, 1024, 1536, 2048, 3072]
    ms = [1, 7, 16, 31, 32, 33, 48, 64, 65, 100, 128, 129, 200, 256, 257, 300, 512, 513, 600]
    ns = [8, 24, 32, 33, 64, 100, 256, 264, 520, 1000, 2048, 4160]
    for it in range(40):
        M, N, K = int(rng.choice(ms)), int(rng.choice(ns)), int(rng.choice(ks))
        fa, fb = (2, 2) if it % 3 else (3, 2)
        la = int(rng.integers(0, 2)) if (M % 32 == 0 and K % 128 == 0) else 0
        lb = int(rng.integers(0, 2)) if (N % 32 == 0 and K % 128 == 0) else 0
        ap, asc, bp, bsc = operands(M, N, K, fa, fb, seed=1000 + it, kind_b="weights")
        ref = gemm(hk, ap, bp, asc, bsc, fa, fb, kernel=1)
        A = hk.tile_operand(dev(ap)) if la else dev(ap)
        B = hk.tile_operand(dev(bp)) if lb else dev(bp)
        As = hk.tile_scales(dev(asc), K) if la else dev(asc)
        Bs = hk.tile_scales(dev(bsc), K) if lb else dev(bsc)
        C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        hk.dispatch_micro(A, B, As, Bs, C, fa, fb, layout_a=la, layout_b=lb)
        torch.cuda.synchronize()
        got = C.cpu().numpy()
        assert np.isfinite(got).all(), (M, N, K, la, lb)
        assert o.rel_err(got, ref) <= TOL_TIGHT, (M, N, K, la, lb, o.rel_err(got, ref))


# ------------------------------------------------------------------ workgroups that walk through several output tiles
@pytest.mark.parametrize("M,N,K,la,lb", [(8192, 8192, 512, 0, 0), (8192, 8192, 768, 0, 0), (8192, 8192, 896, 1, 1), (8192, 8192, 640, 0, 0),
                                         (5000, 5000, 1024, 0, 0), (4352, 4352, 1280, 0, 1), (4128, 8200, 2048, 0, 0), (8192, 16384, 1152, 1, 0),
                                         (100, 264, 640, 0, 0), (1000, 4104, 1280, 0, 0), (2176, 8192, 896, 1, 1)])
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_tiled_kernel_walk_matches_generic_kernel_bit_for_bit(hk, M, N, K, la, lb, out):
    """More output tiles than compute units: every workgroup of the tiled kernel takes several tiles in turn, the loads of
    the next tile running under the last K-tiles of the current one (K-tile counts 4n, 4n+2, 4n+3; 4n+1 keeps one workgroup
    per tile), with ragged edge tiles and tile-major operands, for every tile shape (256 x 256, 128 x 256, 128 x 128).  The result
    must equal the one-wave-per-tile kernel's in every
    bit (both round the same fp32 sums once), and nothing may be written outside C (guard rows before and after it)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(M + N + K)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2, layout=la)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.05, 2, layout=lb)
    prev_r = hk.tk_kernel.set_relayout(0)
    res = []
    try:
        for kern in (1, hk.tk_kernel.KERNEL_TILED_128, hk.tk_kernel.KERNEL_TILED_256, hk.tk_kernel.KERNEL_TILED_128x128):
            full = torch.full((M + 2, N), 12345.0, dtype=out, device="cuda")
            prev = hk.tk_kernel.set_kernel(kern)
            try:
                hk.dispatch_micro(a, b, asc, bsc, full[1:M + 1], 2, 2, layout_a=la, layout_b=lb)
                torch.cuda.synchronize()
            finally:
                hk.tk_kernel.set_kernel(prev)
            res.append(full)
    finally:
        hk.tk_kernel.set_relayout(prev_r)
    ref = res[0]
    for got in res[1:]:
        assert bool((got[0] == 12345.0).all()) and bool((got[-1] == 12345.0).all())
        assert torch.equal(ref[1:-1], got[1:-1])


# ------------------------------------------------------------------ fused epilogue
@pytest.mark.parametrize("kernel,M,N,K", [(1, 70, 40, 96), (3, 16, 96, 1024), (3, 32, 100, 512), (4, 64, 72, 1024), (4, 200, 136, 2048),
                                          (5, 300, 264, 640), (6, 300, 264, 640), (5, 1024, 4104, 512), (6, 2304, 8200, 512),
                                          (17, 300, 264, 640), (17, 1024, 4104, 512), (23, 300, 264, 1024), (24, 200, 136, 2048), (26, 300, 520, 1024), (28, 48, 264, 1024), (28, 200, 136, 8192)])
@pytest.mark.parametrize("activation", [None, "relu", "gelu", "silu"])
def test_fused_epilogue_every_kernel(hk, kernel, M, N, K, activation):
    """act(acc * row_scale * col_scale + bias) fused into each kernel's epilogue (the last two shapes have more tiles than
    CUs: the tiled kernel walks).  The accumulators are the same kernel's unfused fp32 output (bit-exact by the other tests),
    so this isolates the epilogue: fp32 arithmetic against the float64 closed forms.  relu and the affine part are exact to
    fp32 rounding of the terms (2e-5 of max(|ref|, 1 % rms) where scale * acc and bias cancel); silu uses the hardware exp2 / reciprocal and gelu a five-term erf with absolute error 1.5e-7,
    held to 1e-4 of max(|ref|, 1 % rms) (the parity metric).  The bf16 output must be the RNE rounding of the fp32 output."""
    rng = np.random.default_rng(M + N + K + kernel)
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=M + kernel)
    dA, dB, dAs, dBs = dev(ap), dev(bp), dev(asc), dev(bsc)
    bias = rng.standard_normal(N).astype(np.float32) * 3
    rs = (0.5 + rng.random(M)).astype(np.float32)
    cs = (0.25 + rng.random(N)).astype(np.float32) * 0.2
    prev = hk.tk_kernel.set_kernel(kernel)
    prev_r = hk.tk_kernel.set_relayout(0)
    try:
        acc = torch.empty(M, N, dtype=torch.float32, device="cuda")
        hk.dispatch_micro(dA, dB, dAs, dBs, acc)
        for use in ((True, True, True), (True, False, False), (False, True, False), (False, False, True), (False, False, False)):
            if not any(use) and activation is None:
                continue
            kw = dict(bias=dev(bias) if use[0] else None, row_scale=dev(rs) if use[1] else None, col_scale=dev(cs) if use[2] else None,
                      activation=activation)
            C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            hk.dispatch_micro(dA, dB, dAs, dBs, C, **kw)
            ref = o.epilogue_ref(acc.cpu().numpy(), bias if use[0] else None, rs if use[1] else None, cs if use[2] else None, activation)
            got = C.cpu().numpy()
            assert np.isfinite(got).all()
            assert o.rel_err(got, ref) <= (1e-4 if activation in ("gelu", "silu") else 2e-5), (use, o.rel_err(got, ref))
            Cb = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
            hk.dispatch_micro(dA, dB, dAs, dBs, Cb, **kw)
            assert torch.equal(Cb, C.to(torch.bfloat16))
        # bf16 bias: the same as its float value
        b16 = dev(bias).to(torch.bfloat16)
        C1 = torch.empty(M, N, dtype=torch.float32, device="cuda"); C2 = torch.empty_like(C1)
        hk.dispatch_micro(dA, dB, dAs, dBs, C1, bias=b16, activation=activation)
        hk.dispatch_micro(dA, dB, dAs, dBs, C2, bias=b16.float(), activation=activation)
        torch.cuda.synchronize()
        assert torch.equal(C1, C2)
    finally:
        hk.tk_kernel.set_kernel(prev)
        hk.tk_kernel.set_relayout(prev_r)


@pytest.mark.parametrize("kernel,M,N,K", [(0, 16, 96, 1024), (0, 64, 128, 1024), (0, 70, 64, 96), (5, 300, 288, 640), (6, 300, 288, 640),
                                          (5, 1024, 4128, 512), (6, 2304, 8224, 896), (0, 4096, 4096, 8192)])
@pytest.mark.parametrize("fmt_c", [2, 3])
def test_fp6_requantised_output(hk, kernel, M, N, K, fmt_c):
    """The GEMM's result written as the next layer's MXFP6 operand: bit for bit the quantiser applied to the fp32 result of
    the same (fused) call.  Kernels 5 / 6 and the large automatic case quantise the accumulators in the tiled kernel's
    epilogue (edge tiles, more tiles than CUs, the re-layout pre-pass); the small automatic cases run another kernel into
    an fp32 workspace and the quantiser."""
    g = torch.Generator(device="cuda"); g.manual_seed(M + N + K)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.05, 2)
    bias = torch.randn(N, device="cuda", generator=g)
    rs = torch.rand(M, device="cuda", generator=g) + 0.5
    prev = hk.tk_kernel.set_kernel(kernel)
    try:
        for kw in (dict(), dict(bias=bias, row_scale=rs, activation="silu")):
            C = torch.empty(M, N, dtype=torch.float32, device="cuda")
            hk.dispatch_micro(a, b, asc, bsc, C, **kw)
            P = torch.full((M, N // 4 * 3), 0xAA, dtype=torch.uint8, device="cuda")
            S = torch.full((M, N // 32), 0xAA, dtype=torch.uint8, device="cuda")
            hk.dispatch_micro(a, b, asc, bsc, P, C_scale=S, fmt_c=fmt_c, **kw)
            torch.cuda.synchronize()
            ep, es = co.quantise(C.cpu().numpy(), fmt_c)
            assert np.array_equal(S.cpu().numpy(), es)
            assert np.array_equal(P.cpu().numpy(), ep)
    finally:
        hk.tk_kernel.set_kernel(prev)


def test_fused_epilogue_automatic_path_with_relayout(hk):
    """The automatic path of a large row-major problem (pre-pass + walking tiled kernel) carries the epilogue along."""
    M = N = 4096; K = 8192
    g = torch.Generator(device="cuda"); g.manual_seed(5)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.05, 2)
    bias = torch.randn(N, device="cuda", generator=g)
    rs = torch.rand(M, device="cuda", generator=g) + 0.5
    acc = torch.empty(M, N, dtype=torch.float32, device="cuda"); C = torch.empty_like(acc)
    hk.dispatch_micro(a, b, asc, bsc, acc)
    hk.dispatch_micro(a, b, asc, bsc, C, bias=bias, row_scale=rs, activation="relu")
    torch.cuda.synchronize()
    want = torch.relu(torch.addcmul(bias[None, :].expand(M, N), acc, rs[:, None].expand(M, N)))  # fma(acc, rs, bias) like the kernel (cs = 1)
    assert torch.allclose(C, want, rtol=2e-6, atol=1e-5)


# ------------------------------------------------------------------ stream capture
def test_graph_capture_replays_match_eager(hk):
    """A size at which the eager path takes the re-layout pre-pass (workspace from the stream-ordered allocator): under
    capture the library must not allocate, and every replay must reproduce the eager result bit for bit."""
    M = N = K = 8192
    g = torch.Generator(device="cuda")
    g.manual_seed(77)
    sets = []
    for _ in range(2):
        a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
        b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g), 2)
        sets.append((a, b, asc, bsc))
    eager = []
    for a, b, asc, bsc in sets:
        C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        hk.dispatch_micro(a, b, asc, bsc, C)
        eager.append(C)
    torch.cuda.synchronize()
    sa, sb, sas, sbs = (t.clone() for t in sets[0])
    Cg = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hk.dispatch_micro(sa, sb, sas, sbs, Cg)
    for rep in range(4):
        a, b, asc, bsc = sets[rep % 2]
        sa.copy_(a); sb.copy_(b); sas.copy_(asc); sbs.copy_(bsc)
        Cg.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Cg, eager[rep % 2]), f"replay {rep}"
        hk.dispatch_micro(a, b, asc, bsc, torch.empty_like(Cg))   # eager work between replays
        torch.cuda.synchronize()


def test_graph_survives_a_regrown_and_a_released_workspace(hk):
    """A graph that recorded a K split holds the stream's workspace pointer.  A larger eager split on the same stream makes
    the library take a larger workspace, and mxfp6_release_workspaces() gives workspaces back: neither may free the block
    the graph replays into (it stays allocated until the process ends), so every replay still reproduces the eager result."""
    from hipkittensp_amd import _lib
    tk = hk.tk_kernel
    small, large = (128, 512, 8192), (256, 2048, 16384)
    assert tk.kernel_choice(*small, 0, 1) in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT)
    assert tk.kernel_choice(*large, 0, 1) in (tk.CHOICE_BLOCK_K_SPLIT, tk.CHOICE_TILED_K_SPLIT)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)

    def make(M, N, K):
        a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
        b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2, layout=1)
        return a, b, asc, bsc

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        a, b, asc, bsc = make(*small)
        eager = torch.empty(small[0], small[1], dtype=torch.bfloat16, device="cuda")
        hk.dispatch_micro(a, b, asc, bsc, eager, layout_b=1)      # warm-up on the capture stream: the workspace exists
        side.synchronize()
        Cg = torch.zeros_like(eager)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            hk.dispatch_micro(a, b, asc, bsc, Cg, layout_b=1)
        la, lb, las, lbs = make(*large)
        Cl = torch.empty(large[0], large[1], dtype=torch.bfloat16, device="cuda")
        for rep in range(3):
            if rep == 1:
                hk.dispatch_micro(la, lb, las, lbs, Cl, layout_b=1)   # a larger split: the stream's workspace grows
            if rep == 2:
                assert _lib.lib().mxfp6_release_workspaces() == 0
                junk = [torch.full((1 << 22,), 7.0, device="cuda") for _ in range(8)]   # whatever the pool hands out next is overwritten
            Cg.zero_()
            graph.replay()
            side.synchronize()
            assert torch.equal(Cg, eager), f"replay {rep}"
            hk.dispatch_micro(la, lb, las, lbs, Cl, layout_b=1)
            side.synchronize()
        del junk
    torch.cuda.synchronize()


# ------------------------------------------------------------------ torch.library operator
def test_torch_op_and_linear_module(hk):
    from hipkittensp_amd import torch_op

    rng = np.random.default_rng(21)
    w = o.make_source("weights", (160, 1024), rng)
    x = o.make_source("normal", (2, 24, 1024), rng)
    lin = torch_op.MXFP6Linear(dev(w))
    assert lin.layout_w == hk.LAYOUT_TILE
    y = lin(dev(x))
    assert y.shape == (2, 24, 160) and y.dtype == torch.bfloat16
    wp, ws = co.quantise(w, 2)
    xp, xs = co.quantise(x.reshape(48, 1024), 2)
    ref = o.gemm_ref(xp, wp, xs, ws, acc=np.float32)
    got = y.view(torch.int16).cpu().numpy().view(np.uint16).reshape(48, 160)
    assert np.array_equal(got, o.f32_to_bf16_bits(torch.ops.hipkittensp.mxfp6_gemm(dev(xp), dev(wp), dev(xs), dev(ws), 2, 2, 0, 0, True).cpu().numpy()))
    assert o.rel_err(o.bf16_bits_to_f32(got), ref) <= 2 ** -7      # bf16 rounding of an in-tolerance result
    # bias and activation ride in the GEMM's epilogue
    b = rng.standard_normal(160).astype(np.float32)
    lin2 = torch_op.MXFP6Linear(dev(w), bias=dev(b), activation="silu")
    y2 = lin2(dev(x)).float().cpu().numpy().reshape(48, 160)
    want = o.epilogue_ref(ref, bias=b, activation="silu")
    assert o.rel_err(y2, want) <= 2 ** -7
    # from 64 rows on (a whole number of 32-row tiles) the input is quantised tile-major: same bytes regrouped, same result
    x3 = o.make_source("normal", (4, 64, 1024), rng)
    y3 = lin2(dev(x3)).float().cpu().numpy().reshape(256, 160)
    xp3, xs3 = co.quantise(x3.reshape(256, 1024), 2)
    want3 = o.epilogue_ref(o.gemm_ref(xp3, wp, xs3, ws, acc=np.float32), bias=b, activation="silu")
    assert o.rel_err(y3, want3) <= 2 ** -7


# ------------------------------------------------------------------ edge cases
def test_empty_and_degenerate(hk):
    z = lambda *s: torch.zeros(*s, dtype=torch.uint8, device="cuda")
    C = torch.ones(0, 8, dtype=torch.bfloat16, device="cuda")
    hk.dispatch_micro(z(0, 24), z(8, 24), z(0, 1), z(8, 1), C)                 # M == 0: no-op
    C = torch.full((4, 8), 7.0, dtype=torch.bfloat16, device="cuda")
    hk.dispatch_micro(z(4, 0), z(8, 0), z(4, 0), z(8, 0), C)                   # K == 0: zeros
    torch.cuda.synchronize()
    assert float(C.float().abs().max()) == 0.0
    # extreme scales: 2^-127 * 2^-127 underflows to 0, 2^127 stays finite against 2^-100
    ap, asc, bp, bsc = operands(32, 32, 64, 2, 2, seed=5)
    got = gemm(hk, ap, bp, np.zeros_like(asc), np.zeros_like(bsc), kernel=1)
    assert np.all(got == 0)
    got = gemm(hk, ap, bp, np.full_like(asc, 254), np.full_like(bsc, 27), kernel=1)
    ref = o.gemm_ref(ap, bp, np.full_like(asc, 254), np.full_like(bsc, 27), acc=np.float64)
    assert np.isfinite(got).all() and o.rel_err(got, ref) <= TOL


def test_leading_dimensions_fold_into_rows(hk):
    ap, asc, bp, bsc = operands(64, 32, 128, 2, 2, seed=9)
    C = torch.empty(2, 32, 32, dtype=torch.float32, device="cuda")
    hk.dispatch_micro(dev(ap).view(2, 32, -1), dev(bp), dev(asc).view(2, 32, -1), dev(bsc), C)
    torch.cuda.synchronize()
    assert o.rel_err(C.view(64, 32).cpu().numpy(), o.gemm_ref(ap, bp, asc, bsc, acc=np.float64)) <= TOL


def test_short_cut_in_front_of_the_checked_path(hk):
    """dispatch_micro recognises the plain call (2-D contiguous tensors on the current device, no epilogue) and skips
    the per-argument checks: same bytes as the checked path on both layouts and both output types, and every call the
    short cut does not recognise still arrives at the checked path's errors."""
    tk = hk.tk_kernel
    ap, asc, bp, bsc = operands(96, 160, 1024, 3, 2, seed=77)
    A, B, As, Bs = dev(ap), dev(bp), dev(asc), dev(bsc)
    At, Bt, Ast, Bst = tk.tile_operand(A), tk.tile_operand(B), tk.tile_scales(As, 1024), tk.tile_scales(Bs, 1024)
    for dt in (torch.float32, torch.bfloat16):
        for args, la, lb in (((A, B, As, Bs), 0, 0), ((At, Bt, Ast, Bst), 1, 1), ((A, Bt, As, Bst), 0, 1)):
            C0 = torch.full((96, 160), float("nan"), dtype=dt, device="cuda")
            C1 = torch.full((96, 160), float("nan"), dtype=dt, device="cuda")
            hk.dispatch_micro(*args, C0, 3, 2, la, lb)
            tk._dispatch_micro_checked(*args, C1, 3, 2, la, lb)
            torch.cuda.synchronize()
            assert torch.equal(C0, C1) and bool(torch.isfinite(C0.float()).all())
    C = torch.empty(96, 160, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="A_scale"):
        hk.dispatch_micro(A, B, As[:, :16].contiguous(), Bs, C, 3, 2)
    with pytest.raises(RuntimeError, match="contiguous"):
        hk.dispatch_micro(A, B, As, Bs, torch.empty(160, 96, dtype=torch.bfloat16, device="cuda").t(), 3, 2)
    with pytest.raises(RuntimeError, match="tile-major operand needs"):
        hk.dispatch_micro(A[:40].contiguous(), Bt, As[:40].contiguous(), Bst, C[:40].contiguous(), 3, 2, 1, 1)
    with pytest.raises(RuntimeError, match="layout_a / layout_b"):
        hk.dispatch_micro(A, B, As, Bs, C, 3, 2, 2, 0)
    with pytest.raises(RuntimeError, match="C: expected dtype"):
        hk.dispatch_micro(A, B, As, Bs, C.to(torch.float16), 3, 2)
    torch.cuda.synchronize()


# ------------------------------------------------------------------ quantiser: bit exact
@pytest.mark.parametrize("fmt", [2, 3])
@pytest.mark.parametrize("kind", ["normal", "weights", "weights_outliers", "laplace"])
def test_gpu_quantiser_bit_exact(hk, fmt, kind):
    x = o.make_source(kind, (300, 1024), np.random.default_rng(fmt + len(kind)))
    x[0, :32] = 0.0                       # zero block
    x[1, :32] = 0.0; x[1, 3] = 1e-42      # denormal-only block
    x[2, 5] = 3e38                        # huge
    x[3, :64] = np.float32(2.0) ** np.arange(-30, 34, dtype=np.float32)  # powers of two
    tab = o.decode_table(fmt)[:32]
    mids = ((tab[:-1] + tab[1:]) / 2).astype(np.float32)
    x[4, :31] = mids; x[4, 31] = tab[-1]  # exact rounding ties under scale 2^0... (blockmax = max -> scale 1)
    x[5, :31] = -mids * 4; x[5, 31] = tab[-1] * 4
    packed, scales = hk.quantize(dev(x), fmt)
    torch.cuda.synchronize()
    ep, es = co.quantise(x, fmt)
    assert np.array_equal(scales.cpu().numpy(), es)
    assert np.array_equal(packed.cpu().numpy(), ep)
    codes, s2 = o.quantise(x, fmt)
    assert np.array_equal(o.pack_fp6(codes), ep) and np.array_equal(s2, es)
    # bf16 input: the quantisation of the same values widened to fp32, in both layouts
    xb = dev(x[:288]).to(torch.bfloat16)
    ep, es = co.quantise(xb.float().cpu().numpy(), fmt)
    for layout in (0, 1):
        packed, scales = hk.quantize(xb, fmt, layout=layout)
        if layout:
            packed, scales = hk.tile_operand(packed, untile=True), hk.tile_scales(scales, 1024, untile=True)
        assert np.array_equal(scales.cpu().numpy(), es) and np.array_equal(packed.cpu().numpy(), ep)


@pytest.mark.parametrize("M,N,K", [(256, 256, 512), (16, 64, 1024), (64, 96, 1024)])
def test_operands_not_16_byte_aligned_run_on_the_generic_kernel(hk, M, N, K):
    """The fast kernels fetch 16 bytes per lane and need 16-byte aligned operands and scales; pointers that are only
    4-byte aligned are accepted and served by the generic kernel with the same result, and a forced fast kernel refuses
    them instead of issuing misaligned loads."""
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=M + N)
    ref = gemm(hk, ap, bp, asc, bsc, kernel=1)

    def shifted(a, off):
        buf = torch.zeros(a.size + 64, dtype=torch.uint8, device="cuda")
        buf[off:off + a.size] = torch.from_numpy(a.reshape(-1)).cuda()
        v = buf[off:off + a.size].view(a.shape)
        assert v.data_ptr() % 16 == off % 16
        return v

    for which, off in (("A", 4), ("B", 8), ("As", 4), ("Bs", 12)):
        A = shifted(ap, off) if which == "A" else dev(ap)
        B = shifted(bp, off) if which == "B" else dev(bp)
        As = shifted(asc, off) if which == "As" else dev(asc)
        Bs = shifted(bsc, off) if which == "Bs" else dev(bsc)
        C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        hk.dispatch_micro(A, B, As, Bs, C)
        torch.cuda.synchronize()
        assert np.array_equal(C.cpu().numpy(), ref), which
        for forced in ((2,) if K % 128 == 0 and N % 8 == 0 else ()) + ((3,) if M <= 128 and K % 512 == 0 else ()):
            prev = hk.tk_kernel.set_kernel(forced)
            try:
                with pytest.raises(RuntimeError, match="bad shape"):
                    hk.dispatch_micro(A, B, As, Bs, C)
            finally:
                hk.tk_kernel.set_kernel(prev)
    # operands off by 2 bytes are rejected outright
    with pytest.raises(RuntimeError, match="alignment"):
        hk.dispatch_micro(shifted(ap, 2), dev(bp), dev(asc), dev(bsc), torch.empty(M, N, dtype=torch.float32, device="cuda"))


def test_two_threads_launching_into_one_stream_share_the_prepass_workspace_safely(hk):
    """The re-layout pre-pass writes tile-major copies into the stream's workspace and the GEMM behind it reads them: two
    threads that call the operator on the same stream with different operands must each get their own product (the library
    enqueues pre-pass and GEMM of one call without letting another call's pre-pass in between)."""
    import threading

    M = N = 8192
    K = 4096            # large enough for the pre-pass on both operands
    g = torch.Generator(device="cuda")
    g.manual_seed(91)
    sets = []
    for _ in range(2):
        a, sa = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
        b, sb = hk.quantize(torch.randn(N, K, device="cuda", generator=g), 2)
        sets.append((a, b, sa, sb))
    want = []
    for ops in sets:
        C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        hk.dispatch_micro(*ops, C)
        want.append(C)
    torch.cuda.synchronize()
    assert not torch.equal(want[0], want[1])
    outs = [[torch.empty(M, N, dtype=torch.bfloat16, device="cuda") for _ in range(6)] for _ in range(2)]
    errs = []

    def work(t):
        try:
            for C in outs[t]:
                hk.dispatch_micro(*sets[t], C)
        except Exception as e:  # noqa: BLE001
            errs.append(e)

    th = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for x in th:
        x.start()
    for x in th:
        x.join()
    torch.cuda.synchronize()
    assert not errs, errs
    for t in range(2):
        for C in outs[t]:
            assert torch.equal(C, want[t])


def test_measurement_probes_run_and_leave_results_alone(hk):
    """The probe kernels bench.py reports (MFMA-only loop on real operand bytes, read-only stream, the tiled kernel's
    clock stamps, raster override): they run, return plausible counters, and a GEMM with the stamps and a raster override on
    gives the same bits as without."""
    from hipkittensp_amd import _lib

    L = _lib.probes()
    M = N = 512
    K = 1024
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=77)
    a, b, sa, sb = dev(ap), dev(bp), dev(asc), dev(bsc)
    stats = torch.zeros(4, dtype=torch.int32, device="cuda")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    waves = L.mxfp6_probe_mfma(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), M, N, K, 2, 2, 64, sink.data_ptr(), stats.data_ptr(), None)
    torch.cuda.synchronize()
    assert waves > 0 and waves % 8 == 0
    st = stats.cpu().numpy().astype(np.int64)
    assert (st[2] - st[0]) % 2**32 > 64 * 4 * 16 and (st[3] - st[1]) % 2**32 > 0      # at least the MFMA issue time, and real time moved
    assert L.mxfp6_probe_mfma(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), 16, N, K, 2, 2, 64, sink.data_ptr(), stats.data_ptr(), None) == -2
    buf = torch.zeros(64 << 20, dtype=torch.uint8, device="cuda")
    assert L.mxfp6_probe_stream(buf.data_ptr(), buf.numel(), 256, 8, stats.data_ptr(), None) == 0
    assert L.mxfp6_probe_stream(buf.data_ptr(), buf.numel(), 512, 4, stats.data_ptr(), None) == 0
    assert L.mxfp6_probe_stream(buf.data_ptr(), buf.numel() - 8192, 256, 8, stats.data_ptr(), None) == -2
    torch.cuda.synchronize()
    ref = gemm(hk, ap, bp, asc, bsc, kernel=2)   # the operator's own library
    assert L.mxfp6_probe_tiled_clock(stats.data_ptr()) == 0 and L.mxfp6_probe_raster(2, 0) == 0
    try:
        stats.zero_()
        got = gemm_probes_lib(ap, bp, asc, bsc, kernel=2)
        st = stats.cpu().numpy().astype(np.int64)
        assert (st[2] - st[0]) % 2**32 > 8 * 1024 and (st[3] - st[1]) % 2**32 > 0  # eight K-tiles of MFMA work at least
    finally:
        L.mxfp6_probe_tiled_clock(None)
        L.mxfp6_probe_raster(0, 1)
    assert np.array_equal(got, ref)
    # the build with idle clocks added (ablation 8: bf16 output, 256 x 256 tiles) multiplies like the kernel itself
    C8 = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert L.mxfp6_probe_tiled_ablation(8) == 0
    pk = L.mxfp6_set_kernel(6)
    try:
        rc = L.mxfp6_gemm_ex(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), C8.data_ptr(), M, N, K, 2, 2, 0, 0, 0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
    finally:
        L.mxfp6_set_kernel(pk)
        L.mxfp6_probe_tiled_ablation(0)
    assert rc == 0, rc
    assert np.array_equal(C8.view(torch.int16).cpu().numpy().view(np.uint16), o.f32_to_bf16_bits(ref))


@pytest.mark.parametrize("M,N,K,kernel,shares", [(256, 1024, 8192, 2, 8), (300, 520, 8192, 2, 4), (128, 1024, 8192, 22, 8), (200, 1032, 4096 + 128, 22, 3), (128, 384, 8192, 22, 8)])
def test_k_split_order_of_workgroups_does_not_change_the_result(hk, M, N, K, kernel, shares):
    """(tile, share) pairs share by share with an eighth of that order per XCD (the library's own), tile by tile, and with
    no XCD remap at all: the same bits, and the oracle's values.  Workgroup counts that are multiples of eight take the
    remap (32, 24, 64 and 24 here); the fourth shape's 18 tiles x 3 shares do not, and its K % 512 != 0 gives a shorter last share."""
    L = hk._lib.probes()   # the raster override is the measurement build's
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=M + K, kind_b="weights")
    ref = o.gemm_ref(ap, bp, asc, bsc, 2, 2, acc=np.float64)
    prev = L.mxfp6_set_k_split(shares)
    got = {}
    try:
        for xcd in (1, 2, 0):
            assert L.mxfp6_probe_raster(0, xcd) == 0
            got[xcd] = gemm_probes_lib(ap, bp, asc, bsc, kernel=kernel)
    finally:
        L.mxfp6_probe_raster(0, 1)
        L.mxfp6_set_k_split(prev)
    check(got[1], ref, 2, 2, ap, asc, bp, bsc)
    assert np.array_equal(got[1], got[2]) and np.array_equal(got[1], got[0])


# ------------------------------------------------------------------ full-size configurations
def _sampled_check(hk, ap, asc, bp, bsc, fa, fb, kernel, rng, ns=48, band=256):
    """Full-size check of one configuration: a whole band of `band` consecutive rows of the fp32 result (all N columns, so
    every tile column, straddling a tile-row boundary) against the C oracle's dequantise-and-matmul; sampled rows and
    columns against the fp64 oracle; exact scale linearity; bf16 = RNE of the accumulators."""
    M, N = ap.shape[0], bp.shape[0]
    C = torch.empty(M, N, dtype=torch.float32, device="cuda")
    dA, dB, dAs, dBs = dev(ap), dev(bp), dev(asc), dev(bsc)
    prev = hk.tk_kernel.set_kernel(kernel)
    try:
        hk.dispatch_micro(dA, dB, dAs, dBs, C, fa, fb)
        if band and M > band:
            r0 = (M // 2 - band // 2) // 32 * 32 + 32  # not aligned to the 128- or 256-row tiles: the band crosses a tile-row boundary
            full = co.gemm_f32(ap[r0:r0 + band], bp, asc[r0:r0 + band], bsc, fa, fb)
            check(C[r0:r0 + band].cpu().numpy(), full, fa, fb)
        rows = np.sort(rng.choice(M, size=min(ns, M), replace=False))
        cols = np.sort(rng.choice(N, size=min(ns, N), replace=False))
        ref = o.gemm_ref(ap[rows], bp[cols], asc[rows], bsc[cols], fa, fb, acc=np.float64)
        got = C[torch.from_numpy(rows).cuda()][:, torch.from_numpy(cols).cuda()].cpu().numpy()
        check(got, ref, fa, fb)
        # exact linearity in the block scales: +1 on every A scale byte doubles every output bit for bit
        C2 = torch.empty_like(C)
        hk.dispatch_micro(dA, dB, dAs + 1, dBs, C2, fa, fb)
        assert torch.equal(C2, 2 * C)
        # bf16 output is the RNE rounding of the accumulators
        Cb = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        hk.dispatch_micro(dA, dB, dAs, dBs, Cb, fa, fb)
        assert torch.equal(Cb, C.to(torch.bfloat16))
        torch.cuda.synchronize()
    finally:
        hk.tk_kernel.set_kernel(prev)
    return C


def test_cfg1_square_8192(hk):
    M = N = K = 8192
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=1)
    C = _sampled_check(hk, ap, asc, bp, bsc, 2, 2, 0, np.random.default_rng(1))
    # operand swap = transpose (the two operands take different paths through the kernel)
    Ct = torch.empty(N, M, dtype=torch.float32, device="cuda")
    hk.dispatch_micro(dev(bp), dev(ap), dev(bsc), dev(asc), Ct, 2, 2)
    torch.cuda.synchronize()
    d = (Ct.t() - C).abs().max().item()
    assert d <= 1e-4 * C.abs().max().item()
    # tiled kernel agrees with the independent generic kernel on a 1024-row band
    prev = hk.tk_kernel.set_kernel(1)
    Cg = torch.empty(1024, N, dtype=torch.float32, device="cuda")
    hk.dispatch_micro(dev(ap[:1024]), dev(bp), dev(asc[:1024]), dev(bsc), Cg, 2, 2)
    torch.cuda.synchronize()
    hk.tk_kernel.set_kernel(prev)
    assert (Cg - C[:1024]).abs().max().item() <= 1e-4 * C.abs().max().item()


def test_cfg2_prefill_outliers(hk):
    M, N, K = 4096, 28672, 8192
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=2, kind_a="normal", kind_b="weights_outliers")
    assert int(bsc.max()) - int(bsc.min()) >= 3      # the outliers widen the E8M0 range
    _sampled_check(hk, ap, asc, bp, bsc, 2, 2, 0, np.random.default_rng(2))


def test_cfg3_decode_skinny(hk):
    M, N, K = 16, 8192, 28672
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=3, kind_a="normal", kind_b="weights")
    _sampled_check(hk, ap, asc, bp, bsc, 2, 2, 0, np.random.default_rng(3), ns=64)
    ref = o.gemm_ref(ap, bp[:256], asc, bsc[:256], acc=np.float64)
    for kernel in (1, 3):  # generic and skinny kernels against the full first 256 columns
        got = gemm(hk, ap, bp[:256], asc, bsc[:256], kernel=kernel)
        check(got, ref, 2, 2)


@pytest.mark.parametrize("M", [64, 128, 256])
def test_batched_decode_full_size(hk, M):
    """cfg3's weights against 64, 128 and 256 rows of A.  The automatic path takes the skinny kernel for 64 rows against
    row-major weights (two accumulator tiles per wave) and the tiled kernel with K split between workgroups otherwise; the
    skinny kernel (for 128 rows: four accumulator tiles, half chunks) is forced as well.  Sampled rows and columns against the fp64
    oracle, the first 256 columns in full, and the whole result against the generic kernel; row-major and tile-major weights."""
    N, K = 8192, 28672
    ap, asc, bp, bsc = operands(M, N, K, 2, 2, seed=30 + M, kind_a="normal", kind_b="weights")
    _sampled_check(hk, ap, asc, bp, bsc, 2, 2, 0, np.random.default_rng(M), ns=64)
    ref = o.gemm_ref(ap, bp[:256], asc, bsc[:256], acc=np.float64)
    check(gemm(hk, ap, bp[:256], asc, bsc[:256], kernel=3 if M <= 128 else 0), ref, 2, 2)
    a, b, sa, sb = dev(ap), dev(bp), dev(asc), dev(bsc)
    full = torch.empty(M, N, dtype=torch.float32, device="cuda")
    prev = hk.tk_kernel.set_kernel(1)
    try:
        hk.dispatch_micro(a, b, sa, sb, full)
    finally:
        hk.tk_kernel.set_kernel(prev)
    bt, sbt = hk.tile_operand(b), hk.tile_scales(sb, K)
    for kernel in ((0, 3) if M <= 128 else (0,)):
        prev = hk.tk_kernel.set_kernel(kernel)
        try:
            for B, Bs, lb in ((b, sb, 0), (bt, sbt, 1)):
                C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
                hk.dispatch_micro(a, B, sa, Bs, C, layout_b=lb)
                torch.cuda.synchronize()
                assert o.rel_err(C.cpu().numpy(), full.cpu().numpy()) <= TOL_TIGHT, (kernel, lb)
        finally:
            hk.tk_kernel.set_kernel(prev)


def test_cfg4_mixed_formats(hk):
    M, N, K = 8192, 8192, 16384
    ap, asc, bp, bsc = operands(M, N, K, 3, 2, seed=4, kind_a="laplace", kind_b="weights")
    _sampled_check(hk, ap, asc, bp, bsc, 3, 2, 0, np.random.default_rng(4))
