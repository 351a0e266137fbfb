"""ctypes binding of libmxfp6_gemm.so (the C ABI declared in include/mxfp6_gemm.h).

The library is loaded from this package's directory and nowhere else.  There is no fallback: if
the shared object has not been built (python -m hipkittensp_amd.build) the import of the operator
fails with an explicit error.  probes() loads libmxfp6_probes.so, the measurement build of the same
sources (include/mxfp6_probes.h): benchmarks and tests of the probes use it, the operator never does.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmxfp6_gemm.so")
PROBES_LIB_PATH = os.path.join(_HERE, "libmxfp6_probes.so")

_lib = None
_probes = None


class Mxfp6LibraryMissing(RuntimeError):
    pass


def _load(path: str) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise Mxfp6LibraryMissing(
            f"{path} is not built; run `python -m hipkittensp_amd.build` (needs hipcc, no GPU). "
            "There is no CPU or PyTorch fallback for the MXFP6 GEMM."
        )
    return ctypes.CDLL(path)


def _bind(L: ctypes.CDLL) -> ctypes.CDLL:
    """Argument types of everything include/mxfp6_gemm.h declares."""
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.mxfp6_gemm.restype = ci
    L.mxfp6_gemm.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    L.mxfp6_gemm_f32out.restype = ci
    L.mxfp6_gemm_f32out.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    L.mxfp6_quantize.restype = ci
    L.mxfp6_quantize.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    L.mxfp6_gemm_ex.restype = ci
    L.mxfp6_gemm_ex.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp]
    L.mxfp6_gemm_fused.restype = ci
    L.mxfp6_gemm_fused.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp, ci, vp, vp, ci, vp]
    L.mxfp6_gemm_fused_fp6.restype = ci
    L.mxfp6_gemm_fused_fp6.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp, ci, vp, vp, ci, vp]
    L.mxfp6_quantize_ex.restype = ci
    L.mxfp6_quantize_ex.argtypes = [vp, vp, vp, ci, ci, ci, ci, vp]
    L.mxfp6_quantize_bf16.restype = ci
    L.mxfp6_quantize_bf16.argtypes = [vp, vp, vp, ci, ci, ci, ci, vp]
    L.mxfp6_tile_operand.restype = ci
    L.mxfp6_tile_operand.argtypes = [vp, vp, ci, ci, ci, vp]
    L.mxfp6_set_relayout.restype = ci
    L.mxfp6_set_relayout.argtypes = [ci]
    L.mxfp6_tile_scales.restype = ci
    L.mxfp6_tile_scales.argtypes = [vp, vp, ci, ci, ci, vp]
    L.mxfp6_set_kernel.restype = ci
    L.mxfp6_set_kernel.argtypes = [ci]
    L.mxfp6_gemm_noalloc.restype = ci
    L.mxfp6_gemm_noalloc.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
    L.mxfp6_blob_bytes.restype = ctypes.c_size_t
    L.mxfp6_blob_bytes.argtypes = [ci, ci]
    L.mxfp6_blob_header_write.restype = ci
    L.mxfp6_blob_header_write.argtypes = [vp, ci, ci, ci]
    L.mxfp6_blob_header_read.restype = ci
    L.mxfp6_blob_header_read.argtypes = [vp, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ci)]
    L.mxfp6_blob_pack.restype = ci
    L.mxfp6_blob_pack.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    L.mxfp6_blob_unpack.restype = ci
    L.mxfp6_blob_unpack.argtypes = [vp, vp, vp, ci, ci, vp]
    L.mxfp6_allow_e3m2_pair.restype = ci
    L.mxfp6_allow_e3m2_pair.argtypes = [ci]
    L.mxfp6_set_k_split.restype = ci
    L.mxfp6_set_k_split.argtypes = [ci]
    L.mxfp6_kernel_choice.restype = ci
    L.mxfp6_kernel_choice.argtypes = [ci, ci, ci, ci]
    L.mxfp6_release_workspaces.restype = ci
    L.mxfp6_release_workspaces.argtypes = []
    L.mxfp6_strerror.restype = ctypes.c_char_p
    L.mxfp6_strerror.argtypes = [ci]
    L.mxfp6_abi_version.restype = ci
    L.mxfp6_abi_version.argtypes = []
    return L


def lib() -> ctypes.CDLL:
    """The operator's library."""
    global _lib
    if _lib is None:
        _lib = _bind(_load(LIB_PATH))
    return _lib


def probes() -> ctypes.CDLL:
    """The measurement build: everything lib() has (its own copy of it) plus the entry points of include/mxfp6_probes.h."""
    global _probes
    if _probes is None:
        L = _bind(_load(PROBES_LIB_PATH))
        vp, ci = ctypes.c_void_p, ctypes.c_int
        L.mxfp6_probe_mfma.restype = ci
        L.mxfp6_probe_mfma.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp, vp, vp]
        L.mxfp6_probe_stream.restype = ci
        L.mxfp6_probe_stream.argtypes = [vp, ctypes.c_size_t, ci, ci, vp, vp]
        L.mxfp6_probe_tiled_clock.restype = ci
        L.mxfp6_probe_tiled_clock.argtypes = [vp]
        L.mxfp6_tile_order.restype = ci
        L.mxfp6_tile_order.argtypes = [ci, ci, ci, ci, vp]
        L.mxfp6_probe_tiled_ablation.restype = ci
        L.mxfp6_probe_tiled_ablation.argtypes = [ci]
        L.mxfp6_probe_raster.restype = ci
        L.mxfp6_probe_raster.argtypes = [ci, ci]
        L.mxfp6_probe_ksplit_plan.restype = ci
        L.mxfp6_probe_ksplit_plan.argtypes = [ci, ci, ci, ci, ci, ctypes.POINTER(ci)]
        L.mxfp6_probe_block.restype = ci
        L.mxfp6_probe_block.argtypes = [ci]
        L.mxfp6_probe_candidate.restype = ci
        L.mxfp6_probe_candidate.argtypes = [ci] * 6 + [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ci)]
        L.mxfp6_probe_time_gemm.restype = ci
        L.mxfp6_probe_time_gemm.argtypes = [vp] * 5 + [ci] * 9 + [ctypes.c_size_t, ctypes.c_size_t, ci, ci, ctypes.POINTER(ctypes.c_double), vp]
        _probes = L
    return _probes


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: {lib().mxfp6_strerror(rc).decode()} (code {rc})")
