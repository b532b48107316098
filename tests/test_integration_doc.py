"""The reference-side binding that the integration notes at the repository root show (their
section 3: a ctypes stub over the C ABI) is executed as written and checked against the CPU
checker: the stub a maintainer would paste must actually work."""
import os
import re

import pytest
import torch

import oracle
from parity import scale_error

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _stub_source():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    section = text[text.index("## 3."):text.index("## 4.")]
    blocks = re.findall(r"```python\n(.*?)```", section, flags=re.S)
    assert len(blocks) == 1, "section 3 holds exactly one python block"
    return blocks[0]


def test_stub_is_present_and_names_the_library():
    src = _stub_source()
    assert "ctypes.CDLL" in src and "ftc_causal_dot_product" in src
    compile(src, "INTEGRATION.md#3", "exec")


@pytest.mark.gpu
def test_stub_runs_and_matches_the_checker():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU")
    from fast_transformers_amd import _native
    src = _stub_source().replace("/path/to/libftc_causal.so", _native.LIB_PATH)
    ns = {}
    exec(compile(src, "INTEGRATION.md#3", "exec"), ns)
    N, H, L, E, M = 2, 4, 700, 64, 64
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=91)
    Qd, Kd, Vd, Gd = (t.cuda() for t in (Q, K, V, G))
    product = torch.zeros(N, H, L, M, device="cuda")
    ns["causal_dot_product_cuda"](Qd, Kd, Vd, product)
    assert scale_error(product.cpu(), oracle.forward(Q, K, V)) <= 1e-4
    grads = [torch.zeros_like(t) for t in (Qd, Kd, Vd)]
    # the gradient arrives expanded (stride 0) after .sum().backward(): the stub must cope
    ns["causal_dot_backward_cuda"](Qd, Kd, Vd, Gd[:1, :1, :1, :1].expand(N, H, L, M), *grads)
    ones_like_g = Gd[:1, :1, :1, :1].expand(N, H, L, M).contiguous().cpu()
    for got, ref in zip(grads, oracle.backward(Q, K, V, ones_like_g)):
        assert scale_error(got.cpu(), ref) <= 1e-4
