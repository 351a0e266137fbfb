"""CPU-side checks of the drop-in boundary: the C ABI library exports what include/mxfp6_gemm.h declares,
and the Python operator rejects bad arguments the way the reference's binding does (RuntimeError,
include/pyutils/pyutils.cuh:22-46).  No kernel is launched here."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mxfp6_gemm.h")
PROBES_HEADER = os.path.join(ROOT, "include", "mxfp6_probes.h")
LIB = os.path.join(ROOT, "hipkittensp_amd", "libmxfp6_gemm.so")
PROBES_LIB = os.path.join(ROOT, "hipkittensp_amd", "libmxfp6_probes.so")


def _declared_functions(header=HEADER):
    src = open(header).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(mxfp6_[a-z0-9_]+)\s*\(", src)))


@pytest.fixture(scope="module")
def built_lib():
    if not os.path.exists(LIB) or not os.path.exists(PROBES_LIB):
        from hipkittensp_amd import build
        build.build(verbose=False)
    return LIB


def test_header_declares_the_operator():
    names = _declared_functions()
    for want in ("mxfp6_gemm", "mxfp6_gemm_f32out", "mxfp6_gemm_ex", "mxfp6_gemm_fused", "mxfp6_gemm_fused_fp6", "mxfp6_quantize", "mxfp6_quantize_ex", "mxfp6_quantize_bf16", "mxfp6_tile_operand", "mxfp6_tile_scales",
                 "mxfp6_strerror", "mxfp6_abi_version", "mxfp6_set_kernel", "mxfp6_set_relayout", "mxfp6_gemm_noalloc", "mxfp6_release_workspaces",
                 "mxfp6_set_k_split", "mxfp6_kernel_choice"):
        assert want in names
    # the operator's header is the operator: measurement entry points live in mxfp6_probes.h
    assert not [n for n in names if "probe" in n] and len(names) <= 25, names
    assert {"mxfp6_probe_mfma", "mxfp6_probe_stream", "mxfp6_probe_tiled_clock", "mxfp6_probe_tiled_ablation", "mxfp6_probe_raster", "mxfp6_tile_order"} <= set(_declared_functions(PROBES_HEADER))


def test_header_compiles_as_plain_c(tmp_path):
    c = tmp_path / "t.c"
    c.write_text('#include "mxfp6_gemm.h"\n#include "mxfp6_probes.h"\nint main(void){return MXFP6_FMT_E2M3 + MXFP6_FMT_E3M2 == 5 ? 0 : 1;}\n')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(c), "-o", str(tmp_path / "t.o")])


def test_library_exports_every_declared_symbol(built_lib):
    out = subprocess.check_output(["nm", "-D", "--defined-only", built_lib], text=True)
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    for name in _declared_functions():
        assert name in exported, f"{name} declared in the header but not exported"
    # ... and nothing else: no measurement entry point is part of the operator's library
    assert {n for n in exported if n.startswith("mxfp6_")} == set(_declared_functions())
    out = subprocess.check_output(["nm", "-D", "--defined-only", PROBES_LIB], text=True)
    exported_probes = {l.split()[-1] for l in out.splitlines() if " T " in l}
    for name in _declared_functions() + _declared_functions(PROBES_HEADER):
        assert name in exported_probes, f"{name} not exported by the measurement build"
    L = ctypes.CDLL(built_lib)          # loads without a GPU
    L.mxfp6_abi_version.restype = ctypes.c_int
    assert L.mxfp6_abi_version() == 200
    L.mxfp6_strerror.restype = ctypes.c_char_p
    L.mxfp6_strerror.argtypes = [ctypes.c_int]
    assert L.mxfp6_strerror(0) == b"success"
    assert b"multiple of 32" in L.mxfp6_strerror(-2) or b"K % 32" in L.mxfp6_strerror(-2)
    assert L.mxfp6_strerror(-12345)  # never NULL


def test_abi_argument_validation_without_a_gpu(built_lib):
    """Shape / format errors are reported before any HIP call, so they are testable on a CPU box."""
    L = ctypes.CDLL(built_lib)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.mxfp6_gemm.restype = ci
    L.mxfp6_gemm.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    one = ctypes.c_void_p(256)
    assert L.mxfp6_gemm(one, one, one, one, one, 16, 16, 48, 2, 2, None) == -2   # K % 32
    assert L.mxfp6_gemm(one, one, one, one, one, -1, 16, 32, 2, 2, None) == -2
    assert L.mxfp6_gemm(one, one, one, one, one, 16, 16, 32, 1, 2, None) == -3   # fp8 code is not ours
    assert L.mxfp6_gemm(one, one, one, one, one, 16, 16, 32, 2, 4, None) == -3
    assert L.mxfp6_gemm(None, one, one, one, one, 16, 16, 32, 2, 2, None) == -1
    assert L.mxfp6_gemm(one, one, one, one, None, 16, 16, 32, 2, 2, None) == -1
    assert L.mxfp6_gemm(ctypes.c_void_p(258), one, one, one, one, 16, 16, 32, 2, 2, None) == -4
    assert L.mxfp6_gemm(one, one, one, one, one, 0, 16, 32, 2, 2, None) == 0     # empty problem: no-op
    L.mxfp6_quantize.restype = ci
    L.mxfp6_quantize.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    assert L.mxfp6_quantize(one, one, one, 4, 40, 2, None) == -2
    assert L.mxfp6_quantize(one, one, one, 4, 64, 5, None) == -3
    assert L.mxfp6_quantize(one, one, one, 0, 64, 2, None) == 0
    L.mxfp6_gemm_ex.restype = ci
    L.mxfp6_gemm_ex.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp]
    assert L.mxfp6_gemm_ex(one, one, one, one, one, 32, 32, 128, 2, 2, 2, 0, 0, None) == -6      # unknown layout
    assert L.mxfp6_gemm_ex(one, one, one, one, one, 48, 32, 128, 2, 2, 1, 0, 0, None) == -2      # tile-major rows % 32
    assert L.mxfp6_gemm_ex(one, one, one, one, one, 32, 32, 96, 2, 2, 0, 1, 0, None) == -2       # tile-major K % 128
    L.mxfp6_gemm_fused.restype = ci
    L.mxfp6_gemm_fused.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp, ci, vp, vp, ci, vp]
    assert L.mxfp6_gemm_fused(one, one, one, one, one, 32, 32, 128, 2, 2, 0, 0, 0, None, 0, None, None, 4, None) == -7   # unknown activation
    assert L.mxfp6_gemm_fused(one, one, one, one, one, 32, 32, 128, 2, 2, 0, 0, 0, ctypes.c_void_p(264), 0, None, None, 0, None) == -4  # float bias 16 B
    assert L.mxfp6_gemm_fused(one, one, one, one, one, 32, 32, 128, 2, 2, 0, 0, 0, None, 0, None, ctypes.c_void_p(260), 0, None) == -4  # col_scale 16 B
    assert L.mxfp6_gemm_fused(one, one, one, one, one, 32, 32, 96, 2, 2, 0, 1, 0, None, 0, None, None, 0, None) == -2    # the checks of gemm_ex
    assert L.mxfp6_gemm_fused(one, one, one, one, one, 0, 32, 128, 2, 2, 0, 0, 0, None, 0, None, None, 1, None) == 0
    L.mxfp6_tile_operand.restype = ci
    L.mxfp6_tile_operand.argtypes = [vp, vp, ci, ci, ci, vp]
    assert L.mxfp6_tile_operand(one, one, 33, 128, 1, None) == -2
    assert L.mxfp6_tile_operand(one, None, 32, 128, 1, None) == -1
    L.mxfp6_tile_scales.restype = ci
    L.mxfp6_tile_scales.argtypes = [vp, vp, ci, ci, ci, vp]
    assert L.mxfp6_tile_scales(one, one, 32, 96, 1, None) == -2
    assert L.mxfp6_tile_scales(None, one, 32, 128, 1, None) == -1
    assert L.mxfp6_tile_scales(one, one, 0, 128, 1, None) == 0
    # the entry point that allocates nothing: the same checks, and only the splits the skinny kernel has
    L.mxfp6_gemm_noalloc.restype = ci
    L.mxfp6_gemm_noalloc.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
    assert L.mxfp6_gemm_noalloc(one, one, one, one, one, 16, 16, 48, 2, 2, 0, None) == -2
    assert L.mxfp6_gemm_noalloc(one, one, one, one, one, 16, 16, 512, 2, 2, 3, None) == -2
    assert L.mxfp6_gemm_noalloc(None, one, one, one, one, 16, 16, 512, 2, 2, 0, None) == -1
    assert L.mxfp6_gemm_noalloc(one, one, one, one, one, 0, 16, 512, 2, 2, 8, None) == 0
    L.mxfp6_strerror.restype = ctypes.c_char_p
    L.mxfp6_strerror.argtypes = [ci]
    assert b"scratch" in L.mxfp6_strerror(-8)
    # kernel override: per thread, unknown codes are an error
    L.mxfp6_set_kernel.restype = ci
    L.mxfp6_set_kernel.argtypes = [ci]
    assert L.mxfp6_set_kernel(99) == -9 and L.mxfp6_set_kernel(-1) == -9
    # measurement switches validate their argument too (they only set per-thread state: no GPU needed)
    P = ctypes.CDLL(PROBES_LIB)
    assert P.mxfp6_probe_tiled_ablation(5) == -2 and P.mxfp6_probe_tiled_ablation(7) == -2 and P.mxfp6_probe_tiled_ablation(9) == -2 and P.mxfp6_probe_tiled_ablation(0) == 0
    assert L.mxfp6_set_k_split(65) == -2 and L.mxfp6_set_k_split(-2) == -2
    prev = L.mxfp6_set_k_split(1)
    assert prev == 0 and L.mxfp6_set_k_split(0) == 1
    L.mxfp6_kernel_choice.restype = ci
    L.mxfp6_kernel_choice.argtypes = [ci, ci, ci, ci]
    assert L.mxfp6_kernel_choice(0, 16, 512, 0) == -2 and L.mxfp6_kernel_choice(16, 16, 48, 0) == -2    # shape
    assert L.mxfp6_kernel_choice(16, 16, 512, 4) == -6 and L.mxfp6_kernel_choice(40, 64, 512, 1) == -2  # layouts; tile-major needs rows % 32
    # e3m2 x e3m2 needs the caller's consent (it can miss the accuracy bar); the check comes before any HIP call
    assert L.mxfp6_gemm(one, one, one, one, one, 16, 16, 512, 3, 3, None) == -12 and b"e3m2 x e3m2" in L.mxfp6_strerror(-12)
    assert L.mxfp6_allow_e3m2_pair(1) == 0 and L.mxfp6_gemm(one, one, one, one, one, 0, 16, 512, 3, 3, None) == 0 and L.mxfp6_allow_e3m2_pair(0) == 1
    # the entry point that allocates nothing: nsplit = 1 is "never split", whatever the shape; 2, 4, 8 need a decode shape
    assert L.mxfp6_gemm_noalloc(one, one, one, one, one, 0, 16, 640, 2, 2, 1, None) == 0
    assert L.mxfp6_set_kernel(2) == 0
    import threading
    seen = []
    th = threading.Thread(target=lambda: seen.append(L.mxfp6_set_kernel(0)))
    th.start(); th.join()
    assert seen == [0]                      # another thread does not see this thread's override
    assert L.mxfp6_set_kernel(0) == 2
    L.mxfp6_release_workspaces.restype = ci
    assert L.mxfp6_release_workspaces() == 0   # nothing held: no HIP call is made


def test_python_operator_rejects_like_the_reference():
    import hipkittensp_amd as hk

    u8 = torch.zeros(4, 24, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="expected a torch Tensor"):
        hk.dispatch_micro([1, 2], u8, u8, u8, u8)
    with pytest.raises(RuntimeError, match="GPU device"):
        hk.dispatch_micro(u8, u8, u8, u8, u8)
    with pytest.raises(RuntimeError, match="contiguous"):
        hk.dispatch_micro(torch.zeros(24, 4, dtype=torch.uint8).t(), u8, u8, u8, u8)
    with pytest.raises(RuntimeError, match="at most 4 dimensions"):
        hk.dispatch_micro(torch.empty(1, 1, 1, 4, 24, dtype=torch.uint8, device="meta"), u8, u8, u8, u8)
    with pytest.raises(RuntimeError):
        hk.quantize(torch.zeros(4, 64))


def test_python_shape_checks_on_meta_device():
    """Shape/dtype validation runs before the library is touched: exercise it with meta tensors."""
    import hipkittensp_amd as hk

    def t(*shape, dtype=torch.uint8):
        return torch.empty(*shape, dtype=dtype, device="meta")

    A, B, As, Bs, C = t(8, 96), t(16, 96), t(8, 4), t(16, 4), t(8, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="dtype uint8"):
        hk.dispatch_micro(t(8, 96, dtype=torch.int8), B, As, Bs, C)
    with pytest.raises(RuntimeError, match="disagree on K"):
        hk.dispatch_micro(A, t(16, 48), As, Bs, C)
    with pytest.raises(RuntimeError, match="whole number of 32-element blocks"):
        hk.dispatch_micro(t(8, 36), t(16, 36), As, Bs, C)
    with pytest.raises(RuntimeError, match="A_scale"):
        hk.dispatch_micro(A, B, t(8, 3), Bs, C)
    with pytest.raises(RuntimeError, match="B_scale"):
        hk.dispatch_micro(A, B, As, t(15, 4), C)
    with pytest.raises(RuntimeError, match="C: expected shape"):
        hk.dispatch_micro(A, B, As, Bs, t(16, 8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="C: expected dtype"):
        hk.dispatch_micro(A, B, As, Bs, t(8, 16, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="fmt_a / fmt_b"):
        hk.dispatch_micro(A, B, As, Bs, C, fmt_a=0)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from hipkittensp_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.Mxfp6LibraryMissing, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_torch_op_fake_shapes():
    """The registered operator gives shapes and dtypes on meta tensors (no GPU, no library call)."""
    import torch
    from hipkittensp_amd import torch_op  # noqa: F401  (registers torch.ops.hipkittensp.mxfp6_gemm)

    K, N = 1024, 96
    A = torch.empty(3, 5, K // 4 * 3, dtype=torch.uint8, device="meta")
    B = torch.empty(N, K // 4 * 3, dtype=torch.uint8, device="meta")
    As = torch.empty(3, 5, K // 32, dtype=torch.uint8, device="meta")
    Bs = torch.empty(N, 2 * 16, dtype=torch.uint8, device="meta")          # tile-major scales: ceil(K/512) * 16 bytes per row
    C = torch.ops.hipkittensp.mxfp6_gemm(A, B, As, Bs, 2, 2, 0, 1, False)
    assert C.shape == (3, 5, N) and C.dtype == torch.bfloat16
    assert torch.ops.hipkittensp.mxfp6_gemm(A, B, As, Bs, 2, 3, 0, 1, True).dtype == torch.float32
    import pytest
    with pytest.raises(RuntimeError):
        torch.ops.hipkittensp.mxfp6_gemm(A, B, As, Bs[:, :7], 2, 2, 0, 0, False)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr)


@pytest.mark.parametrize("tiles_m,tiles_n", [(1, 1), (1, 7), (7, 1), (3, 5), (4, 8), (32, 32), (16, 112), (5, 13), (33, 31), (9, 9), (2, 3), (61, 7)])
@pytest.mark.parametrize("group_m,xcd", [(4, 1), (4, 0), (1, 1), (8, 1), (16, 1), (3, 1)])
def test_tile_order_is_a_bijection(built_lib, tiles_m, tiles_n, group_m, xcd):
    """The tiled kernel's workgroup -> tile map (XCD remap + grouped raster), evaluated by the library's own function on
    the host: every tile exactly once for ragged tile counts too (the reference's remap leaves tail ids unmapped,
    include/common/util.cuh:92), and with the remap on, the tiles one XCD works on form a contiguous run of the raster."""
    import numpy as np

    L = ctypes.CDLL(PROBES_LIB)
    L.mxfp6_tile_order.restype = ctypes.c_int
    L.mxfp6_tile_order.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p]
    nb = tiles_m * tiles_n
    order = np.full(nb, -7, np.int32)
    assert L.mxfp6_tile_order(tiles_m, tiles_n, group_m, xcd, order.ctypes.data) == 0
    pm, pn = order & 0xFFFF, order >> 16
    assert pm.min() >= 0 and pm.max() < tiles_m and pn.min() >= 0 and pn.max() < tiles_n
    assert len(set(zip(pm.tolist(), pn.tolist()))) == nb                      # a bijection onto the tile grid
    # the raster without the remap: groups of group_m tile rows, columns inside a group, rows fastest
    ident = np.full(nb, -7, np.int32)
    assert L.mxfp6_tile_order(tiles_m, tiles_n, group_m, 0, ident.ctypes.data) == 0
    k = 0
    for first in range(0, tiles_m, group_m):
        gsz = min(group_m, tiles_m - first)
        for col in range(tiles_n):
            for r in range(gsz):
                assert ident[k] == (first + r) | col << 16
                k += 1
    if xcd:
        # workgroups b, b + 8, b + 16, ... (one XCD) get consecutive positions of that raster
        pos = {int(v): i for i, v in enumerate(ident)}
        for x in range(min(8, nb)):
            run = [pos[int(order[b])] for b in range(x, nb, 8)]
            assert run == list(range(run[0], run[0] + len(run)))
        starts = sorted(pos[int(order[x])] for x in range(min(8, nb)))
        assert starts[0] == 0


def test_blob_header_round_trip_and_rejections(built_lib):
    """The 16-byte header of the serialised tile-major operand: written and read on the host, byte for byte as documented."""
    L = ctypes.CDLL(built_lib)
    ci, vp = ctypes.c_int, ctypes.c_void_p
    L.mxfp6_blob_bytes.restype = ctypes.c_size_t
    L.mxfp6_blob_bytes.argtypes = [ci, ci]
    L.mxfp6_blob_header_write.restype = ci
    L.mxfp6_blob_header_write.argtypes = [vp, ci, ci, ci]
    L.mxfp6_blob_header_read.restype = ci
    L.mxfp6_blob_header_read.argtypes = [vp, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ci)]
    assert L.mxfp6_blob_bytes(64, 640) == 16 + 64 * 480 + 64 * 2 * 16      # K = 640: two groups of four K-tiles of scales
    assert L.mxfp6_blob_bytes(8192, 8192) == 16 + 8192 * 6144 + 8192 * 256
    assert L.mxfp6_blob_bytes(33, 128) == 0 and L.mxfp6_blob_bytes(32, 96) == 0
    buf = ctypes.create_string_buffer(16)
    assert L.mxfp6_blob_header_write(buf, 96, 1152, 3) == 0
    assert buf.raw == b"MX6T" + bytes([1, 3, 1, 0]) + (96).to_bytes(4, "little") + (1152).to_bytes(4, "little")
    rows, K, fmt = ci(), ci(), ci()
    assert L.mxfp6_blob_header_read(buf, ctypes.byref(rows), ctypes.byref(K), ctypes.byref(fmt)) == 0
    assert (rows.value, K.value, fmt.value) == (96, 1152, 3)
    assert L.mxfp6_blob_header_write(buf, 96, 100, 2) == -2 and L.mxfp6_blob_header_write(buf, 96, 128, 4) == -3
    good = bytearray(buf.raw)
    for pos, val in ((0, ord("X")), (4, 2), (5, 1), (6, 0), (7, 9), (8, 1), (12, 7)):   # magic, version, fmt, layout, reserved, rows % 32, K % 128
        bad = bytearray(good)
        bad[pos] = val
        assert L.mxfp6_blob_header_read(bytes(bad), ctypes.byref(rows), ctypes.byref(K), ctypes.byref(fmt)) == -10, pos
    L.mxfp6_strerror.restype = ctypes.c_char_p
    L.mxfp6_strerror.argtypes = [ci]
    assert b"blob" in L.mxfp6_strerror(-10)
