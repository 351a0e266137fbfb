"""mxfp6_gemm_noalloc (the entry point that allocates nothing: the K split of decode shapes keeps its partial tiles in a
static array of the library's device code) against mxfp6_gemm, through the C ABI.  Two calls in a row share the array,
the second with a smaller input; then explicit splits, the size limit, and shapes that run on the other kernels.
Collected last (file name), so that a failure here hides no other test."""
import numpy as np
import pytest
import torch

from oracle import mxfp6_oracle as o

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hk():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import hipkittensp_amd as m
    from hipkittensp_amd import _lib

    _lib.lib()  # no fallback: the HIP library must be there
    return m


def _operands(hk, M, N, K, seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
    b, bsc = hk.quantize(torch.randn(N, K, device="cuda", generator=g) * 0.02, 2)
    return a, asc, b, bsc


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _existing(hk, a, asc, b, bsc, kernel=0, dtype=torch.bfloat16):
    C = torch.full((a.shape[0], b.shape[0]), float("nan"), dtype=dtype, device="cuda")
    prev = hk.tk_kernel.set_kernel(kernel)
    try:
        hk.dispatch_micro(a, b, asc, bsc, C)  # mxfp6_gemm's kernels (mxfp6_gemm_fused with nothing fused)
    finally:
        hk.tk_kernel.set_kernel(prev)
    torch.cuda.synchronize()
    return C


def _noalloc(hk, a, asc, b, bsc, nsplit=0):
    C = torch.full((a.shape[0], b.shape[0]), float("nan"), dtype=torch.bfloat16, device="cuda")
    hk.tk_kernel.dispatch_micro_noalloc(a, b, asc, bsc, C, nsplit=nsplit)
    torch.cuda.synchronize()
    return C


def test_two_calls_in_a_row_second_smaller(hk):
    # both shapes are split by the automatic choice (N <= 2048, K >= 24576): the scratch array is in use
    big = _operands(hk, 16, 2048, 28672, 11)
    small = _operands(hk, 16, 512, 24576, 12)
    want_big, want_small = _existing(hk, *big), _existing(hk, *small)
    got_big = _noalloc(hk, *big)
    got_small = _noalloc(hk, *small)  # finds the first call's partial tiles and (cleared) counters in the array
    assert np.array_equal(_bits(got_big), _bits(want_big))
    assert np.array_equal(_bits(got_small), _bits(want_small))
    # and against the generic kernel's accumulators, rounded to bf16, within one bf16 step of an fp32 rounding difference
    for ops, got in ((big, got_big), (small, got_small)):
        ref = _existing(hk, *ops, kernel=1, dtype=torch.float32).cpu().numpy()
        assert o.rel_err(got.float().cpu().numpy(), ref) <= 2.0 ** -8
    # again, the other way round and back to back without a synchronisation between the launches
    C1 = torch.full((16, 512), float("nan"), dtype=torch.bfloat16, device="cuda")
    C2 = torch.full((16, 2048), float("nan"), dtype=torch.bfloat16, device="cuda")
    C3 = torch.full((16, 512), float("nan"), dtype=torch.bfloat16, device="cuda")
    hk.tk_kernel.dispatch_micro_noalloc(small[0], small[2], small[1], small[3], C1)
    hk.tk_kernel.dispatch_micro_noalloc(big[0], big[2], big[1], big[3], C2)
    hk.tk_kernel.dispatch_micro_noalloc(small[0], small[2], small[1], small[3], C3)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(C1), _bits(want_small)) and np.array_equal(_bits(C2), _bits(want_big)) and np.array_equal(_bits(C3), _bits(want_small))


@pytest.mark.parametrize("nsplit", [1, 2, 4, 8])
def test_explicit_split(hk, nsplit):
    ops = _operands(hk, 32, 96, 512 * 24, 20 + nsplit)
    ref = _existing(hk, *ops, kernel=1, dtype=torch.float32).cpu().numpy()
    got = _noalloc(hk, *ops, nsplit=nsplit)
    assert o.rel_err(got.float().cpu().numpy(), ref) <= 2.0 ** -8
    # the same split on the allocating path (forced geometry, 16 rows of B per workgroup: N <= 4096): bit-identical
    if nsplit > 1:
        want = _existing(hk, *ops, kernel={2: 13, 4: 14, 8: 15}[nsplit])
        assert np.array_equal(_bits(got), _bits(want))


def test_limit_and_other_kernels(hk):
    from hipkittensp_amd import _lib

    L = _lib.lib()
    a, asc, b, bsc = _operands(hk, 16, 4096, 1024, 31)
    C = torch.empty(16, 4096, dtype=torch.bfloat16, device="cuda")
    args = (a.data_ptr(), b.data_ptr(), asc.data_ptr(), bsc.data_ptr(), C.data_ptr(), 16, 4096, 1024, 2, 2)
    # 256 tiles of 16 columns x 2 splits = 512 partial tiles > 256
    assert L.mxfp6_gemm_noalloc(*args, 2, None) == -8
    assert b"scratch" in L.mxfp6_strerror(-8)
    assert L.mxfp6_gemm_noalloc(*args, 3, None) == -2  # not a split this kernel has
    torch.cuda.synchronize()
    got = _noalloc(hk, a, asc, b, bsc, nsplit=1)
    assert np.array_equal(_bits(got), _bits(_existing(hk, a, asc, b, bsc)))
    # a split needs the skinny kernel's shapes
    a2, asc2, b2, bsc2 = _operands(hk, 64, 64, 1024, 32)
    C2 = torch.empty(64, 64, dtype=torch.bfloat16, device="cuda")
    assert L.mxfp6_gemm_noalloc(a2.data_ptr(), b2.data_ptr(), asc2.data_ptr(), bsc2.data_ptr(), C2.data_ptr(), 64, 64, 1024, 2, 2, 2, None) == -2
    # shapes of the other kernels run too.  The header promises bit-identity only where both entry points take the same
    # kernel; here mxfp6_gemm may take one the no-allocation path has not (the block kernel, a K split), which adds the same
    # products in another order: equal within one bf16 step of the fp32 result
    for M, N, K, seed in ((64, 64, 1024, 33), (300, 264, 640, 34), (70, 40, 96, 35)):
        ops = _operands(hk, M, N, K, seed)
        got = _noalloc(hk, *ops).float()
        a_, asc_, b_, bsc_ = ops
        ref = torch.empty(M, N, dtype=torch.float32, device="cuda")
        hk.dispatch_micro(a_, b_, asc_, bsc_, ref)
        torch.cuda.synchronize()
        assert torch.all((got - ref).abs() <= ref.abs() * 2.0 ** -7 + 1e-30)
