"""The C-ABI library loads and exports every symbol include/ftc_causal_product.h declares.
No compute call is made here (no GPU needed)."""
import ctypes
import os
import re

import pytest

from fast_transformers_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ftc_causal_product.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ftc_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_entry_points():
    names = declared_functions()
    assert "ftc_causal_dot_product" in names and "ftc_causal_dot_backward" in names
    assert set(names) == set(_native.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_native.LIB_PATH), "build the library first (python fast-transformers_amd/build.py)"
    lib = ctypes.CDLL(_native.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_host_only_calls():
    lib = _native.load()
    assert lib.ftc_version() >= 1000
    assert lib.ftc_causal_dot_product_workspace_bytes(1, 1, 10, 8, 8, _native.FTC_F32) >= 0
    assert lib.ftc_causal_dot_backward_workspace_bytes(10, 8, 1000, 64, 64, _native.FTC_F32) >= 0
    # sizes outside the covered range and bad dtypes are reported, not crashed on
    # (rows of more than 512 values: fp32 in pieces, bf16 refused)
    assert lib.ftc_causal_dot_product_workspace_bytes(1, 1, 10, 4096, 8, _native.FTC_F32) > 0
    assert lib.ftc_causal_dot_product_workspace_bytes(1, 1, 10, 4096, 8, _native.FTC_BF16) == -2
    assert "fp32" in _native.last_error()
    assert lib.ftc_causal_dot_product_workspace_bytes(1, 1, 10, 8, 8, 7) == -1
    assert lib.ftc_causal_dot_product_workspace_bytes(-1, 1, 10, 8, 8, 0) == -1


def test_argument_errors_are_status_codes_not_crashes():
    lib = _native.load()
    t = _native.Tensor4()
    assert lib.ftc_causal_dot_product(None, None, None, None, None, 0, None) == -1
    assert "null" in _native.last_error()
    # a shape mismatch is caught before anything touches a device (pointers never read)
    q = _native.Tensor4(256, 0, (1, 1, 4, 8), (32, 32, 8, 1))
    k = _native.Tensor4(256, 0, (1, 1, 5, 8), (40, 40, 8, 1))
    v = _native.Tensor4(256, 0, (1, 1, 4, 8), (32, 32, 8, 1))
    o = _native.Tensor4(256, 0, (1, 1, 4, 8), (32, 32, 8, 1))
    rc = lib.ftc_causal_dot_product(ctypes.byref(q), ctypes.byref(k), ctypes.byref(v),
                                    ctypes.byref(o), None, 0, None)
    assert rc == -1 and "keys" in _native.last_error()
    del t


def test_python_surface_matches_reference_module():
    from fast_transformers_amd import causal_product as cp
    import torch
    assert issubclass(cp.CausalDotProduct, torch.autograd.Function)
    assert set(cp.CausalDotProduct.dot) == set(cp.CausalDotProduct.dot_backward) == {"cpu", "cuda"}
    assert callable(cp.causal_dot_product)


def test_cpu_entry_matches_the_checker():
    """CPU tensors take the package's own host implementation (the reference keeps a "cpu"
    entry beside "cuda", causal_product/__init__.py:23-30); checked against the CPU checker
    and through autograd."""
    import torch
    import oracle
    from parity import scale_error
    from fast_transformers_amd import causal_product as cp
    Q, K, V, G = oracle.make_inputs(2, 3, 300, 20, 24, seed=5)
    Qg, Kg, Vg = (t.clone().requires_grad_(True) for t in (Q, K, V))
    out = cp.causal_dot_product(Qg, Kg, Vg)
    (out * G).sum().backward()
    assert scale_error(out.detach(), oracle.forward(Q, K, V)) <= 1e-5
    for got, ref in zip((Qg.grad, Kg.grad, Vg.grad), oracle.backward(Q, K, V, G)):
        assert scale_error(got, ref) <= 1e-5
