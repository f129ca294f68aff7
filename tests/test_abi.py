"""CPU checks of the boundary: the C-ABI library loads and exports every declared symbol, the header
and the Python binding agree, and the MEX gateway compiles against the header."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nnvhip.h")
LIB = os.path.join(ROOT, "nnv_amd", "libnnvhip.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nnvhip_[A-Za-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for s in ("nnvhip_create", "nnvhip_star_create", "nnvhip_star_from_box", "nnvhip_affine_fc",
              "nnvhip_affine_conv2d", "nnvhip_relu_relax", "nnvhip_estimate_ranges",
              "nnvhip_star_fetch_constraints", "nnvhip_last_error"):
        assert s in syms


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built (python -m nnv_amd.build)")
def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)          # loading needs the HIP runtime but no GPU
    for s in declared_symbols():
        assert hasattr(lib, s), "libnnvhip.so does not export " + s


def test_python_binding_lists_every_declared_symbol():
    from nnv_amd import _lib
    assert sorted(_lib.SYMBOLS) == declared_symbols()


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built")
def test_no_gpu_is_reported_not_hidden():
    """Without a GPU the context constructor must fail loudly (there is no CPU fallback)."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from nnv_amd import _lib
    with pytest.raises((_lib.NNVHipError, MemoryError, ValueError)):
        _lib.Context(0)


@pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not available")
def test_mex_gateway_compiles_against_the_header():
    src = os.path.join(ROOT, "nnv_amd", "matlab", "nnvhip_mex.cpp")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "tests", "stubs"), src]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert p.returncode == 0, p.stdout
    # the gateway uses every layer/set verb of the ABI
    text = open(src).read()
    for s in ("nnvhip_affine_fc", "nnvhip_affine_conv2d", "nnvhip_relu_relax", "nnvhip_estimate_ranges_batch",
              "nnvhip_star_fetch_constraints", "nnvhip_star_from_box"):
        assert s in text
