"""The C ABI called from a plain-C program: no Python and no torch in the process that makes the calls.

tests/c_host/abi_host.c links the library through include/mxfp6_gemm.h and checks quantiser, fp32 and bf16 outputs and the
entry point that allocates nothing against the C oracle, on the shapes listed there; __graft_entry__.build() compiles
it.  The binary runs as a child of a process that has not touched the GPU itself, which is why this file is named to be
collected before the other GPU tests; when the GPU is already initialised in this process the test is skipped rather
than starting a program from it.
"""
import os
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "c_host", "abi_host")


@pytest.mark.gpu
def test_plain_c_caller_matches_the_oracle():
    if torch.cuda.device_count() < 1:  # counting devices does not initialise the GPU
        pytest.skip("no GPU")
    if torch.cuda.is_initialized():
        pytest.skip("this process has already initialised the GPU: run this file on its own")
    if not os.path.exists(BINARY):
        pytest.skip("tests/c_host/abi_host is not built here: __graft_entry__.build() compiles it")
    r = subprocess.run([BINARY], capture_output=True, text=True, timeout=180)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, f"exit status {r.returncode}\n{r.stdout}\n{r.stderr}"
    assert "ALL OK" in r.stdout and r.stdout.count(" ok") == 6


def test_header_version_is_what_the_library_reports():
    import ctypes
    import re

    from hipkittensp_amd import _lib

    text = open(os.path.join(ROOT, "include", "mxfp6_gemm.h")).read()
    macro = int(re.search(r"#define MXFP6_ABI_VERSION (\d+)", text).group(1))
    L = _lib.lib()
    L.mxfp6_abi_version.restype = ctypes.c_int
    assert L.mxfp6_abi_version() == macro


def test_c_host_source_compiles_against_the_header(tmp_path):
    """Syntax and prototypes only (no link): the calls in abi_host.c match include/mxfp6_gemm.h."""
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                           "-I", "/opt/rocm/include", os.path.join(ROOT, "tests", "c_host", "abi_host.c")])
