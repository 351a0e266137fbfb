"""`tk_kernel` -- the Python-facing operator module, in the reference's calling convention.

The reference builds one pybind11 module named ``tk_kernel`` per kernel and calls
``tk_kernel.dispatch_micro(A, B, C)`` with torch tensors: C = A . B^T, both operands K-contiguous,
C allocated by the caller and written in place, nothing returned, the launch asynchronous
(kernels/gemm/bf16fp32/bench.py:34, kernels/gemm/bf16fp32/utils.py:28-37,
analysis/bf16_gemm/mi325x/kernel_8192.cpp:227-237).  Its binding accepts any object whose type is
named "Tensor", requires it contiguous, on a device and of at most 4 dimensions, and raises
RuntimeError otherwise (include/pyutils/pyutils.cuh:15-48).  This module keeps that behaviour and
adds the checks a packed format needs (dtype, packed width, scale shape).

    dispatch_micro(A, B, A_scale, B_scale, C, fmt_a=2, fmt_b=2)

    A        uint8 [M, 3K/4]   packed fp6, 4 values per 3 bytes, K contiguous
    B        uint8 [N, 3K/4]
    A_scale  uint8 [M, K/32]   E8M0, one per 32-element K-block
    B_scale  uint8 [N, K/32]
    C        bfloat16 [M, N]   (a float32 C receives the accumulators before the bf16 rounding)
    fmt_*    2 = e2m3, 3 = e3m2
    layout_* LAYOUT_ROW (as above) or LAYOUT_TILE: the same bytes regrouped into 32-row x 128-element
             tiles in the kernels' LDS order, with the scales regrouped into 32-row x 16-byte chunks
             (shape [rows, ceil(K/512) * 16]); tile_operand() / tile_scales() convert and
             quantize(..., layout=LAYOUT_TILE) emits both directly; loads of a tile-major operand and
             of its scales are contiguous

PyTorch is used for tensor storage and the current stream only; the work is done by the HIP
library behind include/mxfp6_gemm.h.
"""
from __future__ import annotations

import ctypes

from . import _lib

E2M3 = 2
E3M2 = 3
LAYOUT_ROW = 0
LAYOUT_TILE = 1

KERNEL_AUTO, KERNEL_GENERIC, KERNEL_TILED, KERNEL_SKINNY, KERNEL_MID, KERNEL_TILED_128, KERNEL_TILED_256 = 0, 1, 2, 3, 4, 5, 6
KERNEL_SKINNY_32, KERNEL_SKINNY_16, KERNEL_SKINNY_HALF = 7, 8, 9  # skinny kernel: rows of B per workgroup 32 / 16, or 32 with half the waves
KERNEL_SKINNY_32_SPLIT = (10, 11, 12)  # 32 rows of B, K range split between 2 / 4 / 8 workgroups
KERNEL_SKINNY_16_SPLIT = (13, 14, 15)  # 16 rows of B, likewise
KERNEL_SKINNY_2WAVES = 16  # 32 rows of B, two waves per workgroup (wide N, short K)
KERNEL_TILED_128x128 = 17  # tiled kernel with output tiles of 128 x 128
KERNEL_SKINNY_64 = 19  # skinny kernel with 64 rows of B per workgroup (two tiles of B against every fragment of A), K unsplit
KERNEL_SKINNY_64_SPLIT = (20, 21)  # the same with the K range split between 2 / 4 workgroups
KERNEL_BLOCK = 22  # 128 x 128 tiles, four waves in step: one barrier per K-tile, fragments double-buffered in registers
KERNEL_BLOCK_3SLOTS, KERNEL_BLOCK_6SLOTS = 23, 24  # the same with its operand ring forced to three / six slots
KERNEL_BLOCK_WIDE = 26  # the block kernel with tiles of 128 x 256 and eight waves
KERNEL_RING = 28  # batched decode: a private stream of B per wave, A through a flag-guarded ring, no barrier per K-tile
KERNEL_TILED_4WAVE = 18  # the 4-wave interleaved schedule of the tiled kernel (measurement: never chosen automatically)


def _as_tensor(obj, name: str):
    # same duck typing and error class as the reference binding (include/pyutils/pyutils.cuh:22-46)
    if type(obj).__name__ != "Tensor":
        raise RuntimeError(f"{name}: expected a torch Tensor, got {type(obj).__name__}")
    if not obj.is_contiguous():
        raise RuntimeError(f"{name}: tensor must be contiguous")
    if obj.device.type == "cpu":
        raise RuntimeError(f"{name}: tensor must be on a GPU device")
    if obj.dim() > 4:
        raise RuntimeError(f"{name}: expected at most 4 dimensions, got {obj.dim()}")
    return obj


def _rows_cols(t, name: str):
    # leading dimensions are folded into rows, like the reference's left padding to 4-D
    sh = t.shape
    if len(sh) == 2:
        return sh[0], sh[1]
    if len(sh) < 1:
        raise RuntimeError(f"{name}: expected at least 1 dimension")
    rows = 1
    for d in sh[:-1]:
        rows *= d
    return rows, sh[-1]


def _stream(device=None):
    """The current stream's raw handle on `device` (default: the current device)."""
    import torch

    try:  # the raw handle, without building a Stream object per call
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if device is None or device.index is None else device.index)
    except AttributeError:
        return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """`with _on_device(d)` that costs nothing when d is already the current device (the usual case)."""

    __slots__ = ("ctx",)

    def __init__(self, device):
        import torch

        self.ctx = None if device.index is None or device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def scale_width(K: int, layout: int = LAYOUT_ROW) -> int:
    """Bytes of scales per row: K/32, or ceil(K/512) * 16 for tile-major scales."""
    return K // 32 if layout == LAYOUT_ROW else (K + 511) // 512 * 16


ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU = 0, 1, 2, 3
_ACTS = {None: 0, "none": 0, "relu": 1, "gelu": 2, "silu": 3, 0: 0, 1: 1, 2: 2, 3: 3}


_torch = None
_fast = None  # (Tensor type, uint8, bfloat16, float32, raw-stream getter, current_device, the library's mxfp6_gemm_fused)


def _fast_state():
    global _torch, _fast
    import torch

    _torch = torch
    get_raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if get_raw is None:
        get_raw = lambda index: torch.cuda.current_stream(index).cuda_stream
    _fast = (torch.Tensor, torch.uint8, torch.bfloat16, torch.float32, get_raw, torch.cuda.current_device, _lib.lib().mxfp6_gemm_fused)
    return _fast


def dispatch_micro(A, B, A_scale, B_scale, C, fmt_a: int = E2M3, fmt_b: int = E2M3, layout_a: int = LAYOUT_ROW,
                   layout_b: int = LAYOUT_ROW, bias=None, row_scale=None, col_scale=None, activation=None, C_scale=None,
                   fmt_c: int = E2M3) -> None:
    """C = dq(A) @ dq(B).T (the full description is _dispatch_micro_checked's, which this is a short cut in front of).

    The usual call -- five contiguous 2-D torch tensors of the right dtypes and shapes on the current GPU, no fused
    epilogue -- is recognised here with one read of each tensor's metadata and goes straight to the library (a few
    microseconds of host time, which is what a small GEMM's launch rate is bound by); everything else, including every
    call that is wrong in some way, takes the checked path below, which handles the general cases and raises the
    reference binding's errors."""
    f = _fast or _fast_state()
    T, u8 = f[0], f[1]
    if (bias is None and row_scale is None and col_scale is None and activation is None and C_scale is None
            and type(A) is T and type(B) is T and type(A_scale) is T and type(B_scale) is T and type(C) is T
            and A.dtype is u8 and B.dtype is u8 and A_scale.dtype is u8 and B_scale.dtype is u8):
        cd = C.dtype
        sa, sb, sas, sbs, sc = A.shape, B.shape, A_scale.shape, B_scale.shape, C.shape
        dev = C.get_device()
        if ((cd is f[2] or cd is f[3]) and len(sa) == 2 and len(sb) == 2 and len(sas) == 2 and len(sbs) == 2 and len(sc) == 2
                and dev >= 0 and dev == f[5]() and A.get_device() == dev and B.get_device() == dev
                and A_scale.get_device() == dev and B_scale.get_device() == dev
                and A.is_contiguous() and B.is_contiguous() and A_scale.is_contiguous() and B_scale.is_contiguous() and C.is_contiguous()
                and (fmt_a == 2 or fmt_a == 3) and (fmt_b == 2 or fmt_b == 3) and (layout_a == 0 or layout_a == 1) and (layout_b == 0 or layout_b == 1)):
            M, wa = sa
            N = sb[0]
            K = wa // 3 * 4
            if (wa == sb[1] and wa % 24 == 0 and sc[0] == M and sc[1] == N and sas[0] == M and sbs[0] == N
                    and sas[1] == (K // 32 if layout_a == 0 else (K + 511) // 512 * 16)
                    and sbs[1] == (K // 32 if layout_b == 0 else (K + 511) // 512 * 16)
                    and (layout_a == 0 or (M % 32 == 0 and K % 128 == 0)) and (layout_b == 0 or (N % 32 == 0 and K % 128 == 0))):
                rc = f[6](A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(), C.data_ptr(), M, N, K,
                          fmt_a, fmt_b, layout_a, layout_b, 1 if cd is f[3] else 0, 0, 0, 0, 0, 0, f[4](dev))
                if rc:
                    _lib.check(rc, "dispatch_micro")
                return
    _dispatch_micro_checked(A, B, A_scale, B_scale, C, fmt_a, fmt_b, layout_a, layout_b, bias, row_scale, col_scale, activation, C_scale, fmt_c)


def _dispatch_micro_checked(A, B, A_scale, B_scale, C, fmt_a: int = E2M3, fmt_b: int = E2M3, layout_a: int = LAYOUT_ROW,
                            layout_b: int = LAYOUT_ROW, bias=None, row_scale=None, col_scale=None, activation=None, C_scale=None,
                            fmt_c: int = E2M3) -> None:
    """C = dq(A) @ dq(B).T; optionally fused, in fp32 before the output rounding:
    C = act(acc * row_scale[:, None] * col_scale[None, :] + bias[None, :]) with bias [N] float32 or bfloat16,
    row_scale [M] and col_scale [N] float32, activation one of None / "relu" / "gelu" / "silu".
    With C_scale given, the result is re-quantised to MXFP6 (fmt_c) along N: C is then the packed operand
    uint8 [M, 3N/4] and C_scale its E8M0 bytes uint8 [M, N/32] (N % 32 == 0), ready to be the next GEMM's A."""
    import torch

    A, B = _as_tensor(A, "A"), _as_tensor(B, "B")
    A_scale, B_scale = _as_tensor(A_scale, "A_scale"), _as_tensor(B_scale, "B_scale")
    C = _as_tensor(C, "C")
    for t, name in ((A, "A"), (B, "B"), (A_scale, "A_scale"), (B_scale, "B_scale")):
        if t.dtype != torch.uint8:
            raise RuntimeError(f"{name}: expected dtype uint8, got {t.dtype}")
    fp6_out = C_scale is not None
    if fp6_out:
        C_scale = _as_tensor(C_scale, "C_scale")
        if C.dtype != torch.uint8 or C_scale.dtype != torch.uint8:
            raise RuntimeError("C and C_scale: expected dtype uint8 for the MXFP6 output")
        if fmt_c not in (E2M3, E3M2):
            raise RuntimeError("fmt_c must be 2 (e2m3) or 3 (e3m2)")
    elif C.dtype not in (torch.bfloat16, torch.float32):
        raise RuntimeError(f"C: expected dtype bfloat16 (or float32 for unrounded output), got {C.dtype}")
    if fmt_a not in (E2M3, E3M2) or fmt_b not in (E2M3, E3M2):
        raise RuntimeError("fmt_a / fmt_b must be 2 (e2m3) or 3 (e3m2)")
    if layout_a not in (LAYOUT_ROW, LAYOUT_TILE) or layout_b not in (LAYOUT_ROW, LAYOUT_TILE):
        raise RuntimeError("layout_a / layout_b must be LAYOUT_ROW (0) or LAYOUT_TILE (1)")
    M, wa = _rows_cols(A, "A")
    N, wb = _rows_cols(B, "B")
    if wa != wb:
        raise RuntimeError(f"A and B disagree on K: packed widths {wa} and {wb}")
    if wa % 24:
        raise RuntimeError(f"packed width {wa} is not a whole number of 32-element blocks (24 bytes each)")
    K = wa // 3 * 4
    for rows, lay, name in ((M, layout_a, "A"), (N, layout_b, "B")):
        if lay == LAYOUT_TILE and (rows % 32 or K % 128):
            raise RuntimeError(f"{name}: a tile-major operand needs rows % 32 == 0 and K % 128 == 0")
    for t, rows, lay, name in ((A_scale, M, layout_a, "A_scale"), (B_scale, N, layout_b, "B_scale")):
        want = (rows, scale_width(K, lay))
        if _rows_cols(t, name) != want:
            raise RuntimeError(f"{name}: expected shape [{want[0]}, {want[1]}], got {tuple(t.shape)}")
    if fp6_out:
        if N % 32:
            raise RuntimeError(f"the MXFP6 output needs N % 32 == 0, got N = {N}")
        if _rows_cols(C, "C") != (M, N // 4 * 3) or _rows_cols(C_scale, "C_scale") != (M, N // 32):
            raise RuntimeError(f"C / C_scale: expected shapes [{M}, {N // 4 * 3}] and [{M}, {N // 32}], got {tuple(C.shape)} and {tuple(C_scale.shape)}")
    elif _rows_cols(C, "C") != (M, N):
        raise RuntimeError(f"C: expected shape [{M}, {N}], got {tuple(C.shape)}")
    if activation not in _ACTS:
        raise RuntimeError(f"activation must be None, 'relu', 'gelu' or 'silu', got {activation!r}")
    extras = []
    for t, name, n, dts in ((bias, "bias", N, (torch.float32, torch.bfloat16)), (row_scale, "row_scale", M, (torch.float32,)),
                            (col_scale, "col_scale", N, (torch.float32,))):
        if t is None:
            continue
        t = _as_tensor(t, name)
        if t.dtype not in dts:
            raise RuntimeError(f"{name}: expected dtype {' or '.join(str(d) for d in dts)}, got {t.dtype}")
        if t.dim() != 1 or t.shape[0] != n or not t.is_contiguous():
            raise RuntimeError(f"{name}: expected a contiguous vector of {n} elements, got shape {tuple(t.shape)}")
        extras.append(t)
    if fp6_out:
        extras.append(C_scale)
    dev = C.device
    for t in (A, B, A_scale, B_scale, *extras):
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on one device, got {sorted({str(x.device) for x in (A, B, A_scale, B_scale, C, *extras)})}")
    L = _lib.lib()
    ptr = lambda t: 0 if t is None else t.data_ptr()
    if fp6_out:
        with _on_device(dev):
            rc = L.mxfp6_gemm_fused_fp6(A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(), C.data_ptr(), C_scale.data_ptr(),
                                        M, N, K, fmt_a, fmt_b, layout_a, layout_b, fmt_c, ptr(bias),
                                        int(bias is not None and bias.dtype == torch.bfloat16), ptr(row_scale), ptr(col_scale),
                                        _ACTS[activation], _stream(dev))
        _lib.check(rc, "dispatch_micro")
        return
    with _on_device(dev):
        rc = L.mxfp6_gemm_fused(A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(), C.data_ptr(), M, N, K,
                                fmt_a, fmt_b, layout_a, layout_b, int(C.dtype == torch.float32), ptr(bias),
                                int(bias is not None and bias.dtype == torch.bfloat16), ptr(row_scale), ptr(col_scale),
                                _ACTS[activation], _stream(dev))
    _lib.check(rc, "dispatch_micro")


def quantize(X, fmt: int = E2M3, layout: int = LAYOUT_ROW):
    """fp32 or bf16 [rows, K] on the GPU -> (packed uint8 [rows, 3K/4], scales uint8 [rows, K/32]).
    With layout=LAYOUT_TILE packed bytes and scales are written tile-major (rows % 32 == 0, K % 128 == 0;
    scales [rows, ceil(K/512) * 16], padding zero)."""
    import torch

    X = _as_tensor(X, "X")
    if X.dtype not in (torch.float32, torch.bfloat16):
        raise RuntimeError(f"X: expected dtype float32 or bfloat16, got {X.dtype}")
    if fmt not in (E2M3, E3M2):
        raise RuntimeError("fmt must be 2 (e2m3) or 3 (e3m2)")
    rows, K = _rows_cols(X, "X")
    if K % 32:
        raise RuntimeError(f"K = {K} is not a multiple of 32")
    packed = torch.empty(*X.shape[:-1], K // 4 * 3, dtype=torch.uint8, device=X.device)
    if layout not in (LAYOUT_ROW, LAYOUT_TILE):
        raise RuntimeError("layout must be LAYOUT_ROW (0) or LAYOUT_TILE (1)")
    sw = scale_width(K, layout)
    alloc = torch.zeros if sw != K // 32 else torch.empty  # the quantiser does not write padding bytes
    scales = alloc(*X.shape[:-1], sw, dtype=torch.uint8, device=X.device)
    with _on_device(X.device):
        fn = _lib.lib().mxfp6_quantize_bf16 if X.dtype == torch.bfloat16 else _lib.lib().mxfp6_quantize_ex
        rc = fn(X.data_ptr(), packed.data_ptr(), scales.data_ptr(), rows, K, fmt, layout, _stream())
    _lib.check(rc, "quantize")
    return packed, scales


def tile_operand(packed, untile: bool = False):
    """Row-major packed operand [rows, 3K/4] -> tile-major (same shape, regrouped bytes), or back."""
    import torch

    packed = _as_tensor(packed, "packed")
    if packed.dtype != torch.uint8:
        raise RuntimeError(f"packed: expected dtype uint8, got {packed.dtype}")
    rows, w = _rows_cols(packed, "packed")
    if w % 96 or rows % 32:
        raise RuntimeError("tile-major layout needs rows % 32 == 0 and K % 128 == 0")
    out = torch.empty_like(packed)
    with _on_device(packed.device):
        rc = _lib.lib().mxfp6_tile_operand(packed.data_ptr(), out.data_ptr(), rows, w // 3 * 4, 0 if untile else 1, _stream())
    _lib.check(rc, "tile_operand")
    return out


def tile_scales(scales, K: int, untile: bool = False):
    """Row-major scales [rows, K/32] -> tile-major [rows, ceil(K/512) * 16], or back (K = elements per row)."""
    import torch

    scales = _as_tensor(scales, "scales")
    if scales.dtype != torch.uint8:
        raise RuntimeError(f"scales: expected dtype uint8, got {scales.dtype}")
    rows, w = _rows_cols(scales, "scales")
    if K % 128 or rows % 32:
        raise RuntimeError("tile-major layout needs rows % 32 == 0 and K % 128 == 0")
    src_w, dst_w = (scale_width(K, LAYOUT_TILE), K // 32) if untile else (K // 32, scale_width(K, LAYOUT_TILE))
    if w != src_w:
        raise RuntimeError(f"scales: expected {src_w} bytes per row for K = {K}, got {w}")
    out = torch.empty(*scales.shape[:-1], dst_w, dtype=torch.uint8, device=scales.device)
    with _on_device(scales.device):
        rc = _lib.lib().mxfp6_tile_scales(scales.data_ptr(), out.data_ptr(), rows, K, 0 if untile else 1, _stream())
    _lib.check(rc, "tile_scales")
    return out


def set_relayout(on: bool) -> bool:
    """Switch the re-layout pre-pass of large row-major GEMMs on / off; returns the previous setting."""
    return bool(_lib.lib().mxfp6_set_relayout(1 if on else 0))


def allow_e3m2_pair(allow: bool) -> bool:
    """e3m2 x e3m2 is the one pair of formats whose result can miss the 2e-3 accuracy bar (the scaled MFMA's own sum is
    inexact there, up to 1e-4 of sum |a||b| per output): dispatch_micro raises for it until this thread has accepted that
    with allow_e3m2_pair(True).  Returns the previous setting."""
    return bool(_lib.lib().mxfp6_allow_e3m2_pair(1 if allow else 0))


def set_k_split(shares: int) -> int:
    """K split of the tiled kernel for this thread's later calls (measurement / tests): 0 = where it pays (default), 1 = never,
    -1 = wherever the shape allows it, n > 1 = n workgroups per output tile; returns the previous setting."""
    return _lib.lib().mxfp6_set_k_split(int(shares))


def k_split_plan(M: int, N: int, K: int, layout_a: int = LAYOUT_ROW, shares: int = 0, layout_b: int = LAYOUT_ROW):
    """(workgroups per output tile, rows of A per tile) the tiled kernel's K split would use for this shape; (1, 0) = none.
    A query of the measurement build (libmxfp6_probes.so: the same host code as the operator's)."""
    rows = ctypes.c_int(0)
    n = _lib.probes().mxfp6_probe_ksplit_plan(int(M), int(N), int(K), int(bool(layout_a)) | int(bool(layout_b)) << 1, int(shares), ctypes.byref(rows))
    if n < 0:
        _lib.check(n, "k_split_plan")
    return n, rows.value


CHOICE_TILED_K_SPLIT = 25  # kernel_choice(): the tiled kernel with its K split between workgroups
CHOICE_BLOCK_K_SPLIT = 27  # kernel_choice(): the block kernel with its K split between workgroups


def kernel_choice(M: int, N: int, K: int, layout_a: int = LAYOUT_ROW, layout_b: int = LAYOUT_ROW) -> int:
    """The kernel (KERNEL_* code, or CHOICE_TILED_K_SPLIT / CHOICE_BLOCK_K_SPLIT) the automatic path takes for this shape; launches nothing."""
    n = _lib.lib().mxfp6_kernel_choice(int(M), int(N), int(K), int(bool(layout_a)) | int(bool(layout_b)) << 1)
    if n < 0:
        _lib.check(n, "kernel_choice")
    return n


def set_kernel(which: int) -> int:
    """Force a kernel (KERNEL_*) for measurement / tests; returns the previous setting."""
    return _lib.lib().mxfp6_set_kernel(int(which))


def dispatch_micro_noalloc(A, B, A_scale, B_scale, C, fmt_a: int = E2M3, fmt_b: int = E2M3, nsplit: int = 0) -> None:
    """dispatch_micro for callers that cannot allocate device memory (graph capture, tight serving loops): row-major
    operands, bfloat16 C, no allocation of any kind behind the call.  nsplit = 0 picks the kernel dispatch_micro would
    pick among those that need no workspace (bit-identical result on the decode shapes the skinny kernel takes; elsewhere
    the same products, possibly added in another order); 1, 2, 4 or 8 fixes the K split of the skinny kernel (M <= 32, K % 512 == 0),
    whose partial tiles live in the library's static scratch memory (256 partial tiles: a RuntimeError says so when a
    split does not fit)."""
    import torch

    A, B = _as_tensor(A, "A"), _as_tensor(B, "B")
    A_scale, B_scale = _as_tensor(A_scale, "A_scale"), _as_tensor(B_scale, "B_scale")
    C = _as_tensor(C, "C")
    for t, name in ((A, "A"), (B, "B"), (A_scale, "A_scale"), (B_scale, "B_scale")):
        if t.dtype != torch.uint8:
            raise RuntimeError(f"{name}: expected dtype uint8, got {t.dtype}")
    if C.dtype != torch.bfloat16:
        raise RuntimeError(f"C: expected dtype bfloat16, got {C.dtype}")
    M, wa = _rows_cols(A, "A")
    N, wb = _rows_cols(B, "B")
    if wa != wb or wa % 24:
        raise RuntimeError(f"A and B: packed widths {wa} and {wb} must agree and be whole 32-element blocks (24 bytes)")
    K = wa // 3 * 4
    if _rows_cols(A_scale, "A_scale") != (M, K // 32) or _rows_cols(B_scale, "B_scale") != (N, K // 32) or _rows_cols(C, "C") != (M, N):
        raise RuntimeError("A_scale / B_scale / C: shapes must be [M, K/32], [N, K/32] and [M, N]")
    if len({t.device for t in (A, B, A_scale, B_scale, C)}) != 1:
        raise RuntimeError("all tensors must be on one device")
    with _on_device(C.device):
        rc = _lib.lib().mxfp6_gemm_noalloc(A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(), C.data_ptr(), M, N, K,
                                           fmt_a, fmt_b, int(nsplit), _stream())
    _lib.check(rc, "dispatch_micro_noalloc")


def release_workspaces() -> None:
    """Return every workspace the library holds to the stream-ordered allocator."""
    _lib.check(_lib.lib().mxfp6_release_workspaces(), "release_workspaces")


def pack_weights(packed, scales, fmt: int = E2M3):
    """Row-major packed operand [rows, 3K/4] + scales [rows, K/32] (GPU tensors) -> one uint8 blob on the GPU: 16-byte
    header (magic "MX6T", version, format, layout, rows, K), tile-major operand, tile-major scales.  The blob can be
    copied to the host and stored; unpack_weights() of a blob in GPU memory gives views that dispatch_micro takes as a
    tile-major operand without any conversion."""
    import torch

    packed, scales = _as_tensor(packed, "packed"), _as_tensor(scales, "scales")
    if packed.dtype != torch.uint8 or scales.dtype != torch.uint8:
        raise RuntimeError("packed / scales: expected dtype uint8")
    rows, w = _rows_cols(packed, "packed")
    if w % 96 or rows % 32:
        raise RuntimeError("a tile-major blob needs rows % 32 == 0 and K % 128 == 0")
    K = w // 3 * 4
    if _rows_cols(scales, "scales") != (rows, K // 32):
        raise RuntimeError(f"scales: expected shape [{rows}, {K // 32}], got {tuple(scales.shape)}")
    L = _lib.lib()
    blob = torch.empty(L.mxfp6_blob_bytes(rows, K), dtype=torch.uint8, device=packed.device)
    with _on_device(packed.device):
        rc = L.mxfp6_blob_pack(packed.data_ptr(), scales.data_ptr(), blob.data_ptr(), rows, K, fmt, _stream())
    _lib.check(rc, "pack_weights")
    return blob


def unpack_weights(blob):
    """A blob of pack_weights() (uint8, GPU) -> (operand [rows, 3K/4], scales [rows, ceil(K/512) * 16], fmt): views into the
    blob in tile-major layout, for dispatch_micro(..., layout_b=LAYOUT_TILE).  Raises RuntimeError for anything that is not
    a blob of a version this library reads."""
    import ctypes

    import torch

    blob = _as_tensor(blob, "blob")
    if blob.dtype != torch.uint8 or blob.dim() != 1 or blob.numel() < 16:
        raise RuntimeError("blob: expected a 1-D uint8 tensor of at least 16 bytes")
    L = _lib.lib()
    head = bytes(blob[:16].cpu().tolist())
    rows, K, fmt = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _lib.check(L.mxfp6_blob_header_read(head, ctypes.byref(rows), ctypes.byref(K), ctypes.byref(fmt)), "unpack_weights")
    rows, K, fmt = rows.value, K.value, fmt.value
    if blob.numel() != L.mxfp6_blob_bytes(rows, K):
        raise RuntimeError(f"blob: header says {L.mxfp6_blob_bytes(rows, K)} bytes, tensor has {blob.numel()}")
    nop = rows * (K // 4 * 3)
    return blob[16:16 + nop].view(rows, K // 4 * 3), blob[16 + nop:].view(rows, scale_width(K, LAYOUT_TILE)), fmt
