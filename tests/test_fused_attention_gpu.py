"""ftc_causal_linear_attention: feature map, key-length mask, causal product and normaliser in
one launch, called through the C ABI and checked against

(a) the outputs of the reference's own CausalLinearAttention
    (tests/golden/attention_causal_linear.npz, written by tests/golden/make_encoder_golden.py),
(b) the CPU restatement ``oracle.causal_linear_attention`` (float32 as the reference runs it,
    float64 as the anchor) on seeded inputs: every supported pair of head dimensions,
    chunk and segment boundaries, ragged / zero / over-long key lengths, (N, L, H, X) views,
(c) properties that hold at any size: rows are weighted means of the values seen so far
    (constant values come back unchanged), prefix property, independence of masked keys,
and, at module level, against the composition of separate operator calls that training uses.

Tolerance: 1e-4 relative to the largest magnitude of the chain (fp32 bar of the operator),
and an element-wise violation fraction (1e-5 + 1e-4 |want|) no worse than twice what the
float32 CPU restatement shows against float64, plus 6e-4.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle
from parity import scale_error, violation_fraction

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU")
    from fast_transformers_amd import _native
    return _native.load()


def fused(lib, q, k, v, lengths, eps, out=None):
    """q, k, v: (N, L, H, X) device tensors (any strides the ABI takes); straight C ABI call."""
    from fast_transformers_amd import _native
    N, L, H, E = q.shape
    M = v.shape[3]
    if out is None:
        out = torch.full((N, L, H, M), float("nan"), device=q.device, dtype=torch.float32)
    nbytes = lib.ftc_causal_linear_attention_workspace_bytes(N, H, L, E, M, _native.FTC_F32)
    assert nbytes >= 0, _native.last_error()
    ws = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=q.device)
    d = [_native.describe(t.permute(0, 2, 1, 3)) for t in (q, k, v, out)]
    rc = lib.ftc_causal_linear_attention(
        ctypes.byref(d[0]), ctypes.byref(d[1]), ctypes.byref(d[2]),
        ctypes.c_void_p(lengths.data_ptr()) if lengths is not None else None,
        ctypes.c_float(eps), ctypes.byref(d[3]), ctypes.c_void_p(ws.data_ptr()), nbytes,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, _native.last_error()
    torch.cuda.synchronize()
    assert int(ws[8:12].view(torch.int32).item()) == 0, "a wavefront gave up waiting"
    return out


def inputs(N, L, H, E, M, seed, scale=1.5):
    gen = torch.Generator().manual_seed(seed)
    q = scale * torch.randn(N, L, H, E, generator=gen)
    k = scale * torch.randn(N, L, H, E, generator=gen)
    v = torch.randn(N, L, H, M, generator=gen)
    return q, k, v


def gate(got, q, k, v, lengths, eps):
    """got: (N, L, H, M) on the host."""
    want32 = oracle.causal_linear_attention(q, k, v, lengths, eps)
    want64 = oracle.causal_linear_attention(q.double(), k.double(), v.double(), lengths, eps)
    nhl = lambda t: t.permute(0, 2, 1, 3)
    assert torch.isfinite(got).all()
    assert scale_error(nhl(got), nhl(want32)) <= 1e-4
    assert scale_error(nhl(got), nhl(want64)) <= max(4 * scale_error(nhl(want32), nhl(want64)), 2e-6)
    v_ref = violation_fraction(want32, want64)
    assert violation_fraction(got, want64) <= 2 * v_ref + 6e-4
    assert violation_fraction(got, want32) <= 2 * v_ref + 6e-4


def test_against_the_reference_modules_outputs(lib):
    data = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_causal_linear.npz"))
    q, k, v, y = (torch.from_numpy(data["b_" + x]) for x in ("q", "k", "v", "y"))
    lengths = torch.from_numpy(data["b_lengths"])
    got = fused(lib, q.cuda(), k.cuda(), v.cuda(), lengths.cuda(), float(data["b_eps"])).cpu()
    assert (got - y).abs().max().item() <= 1e-4 * max(1.0, y.abs().max().item())
    assert violation_fraction(got, y) == 0.0


SHAPES = [
    # N, L, H, E, M, key lengths (None: all)
    (2, 1, 2, 64, 64, None),
    (2, 31, 3, 64, 64, [31, 7]),
    (1, 32, 2, 64, 32, [32]),
    (3, 33, 1, 32, 64, [33, 0, 32]),
    (2, 100, 4, 32, 32, [64, 100]),
    (2, 1000, 8, 64, 64, [1000, 517]),
    (1, 4096, 2, 64, 64, [3000]),          # several segments; the length cuts one of them
    (2, 4100, 3, 32, 64, [4100, 33]),      # whole segments beyond the length
    (1, 2500, 5, 64, 32, [9999]),          # longer than the sequence: every key counts
    (3, 777, 2, 32, 32, None),
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "n%d_l%d_h%d_e%d_m%d" % s[:5])
def test_against_the_cpu_restatement(lib, shape):
    N, L, H, E, M, lens = shape
    q, k, v = inputs(N, L, H, E, M, seed=100 + L)
    lengths = torch.tensor(lens) if lens is not None else None
    got = fused(lib, q.cuda(), k.cuda(), v.cuda(),
                lengths.cuda() if lengths is not None else None, 1e-6).cpu()
    gate(got, q, k, v, lengths, 1e-6)


def test_strided_views_and_eps(lib):
    """Rows taken out of wider storage (the fused projection layout of an attention layer)
    and a large eps."""
    N, L, H, E, M = 2, 300, 4, 64, 64
    q, k, v = inputs(N, L, H, E, M, seed=7)
    wide = torch.zeros(N, L, H, 3 * 64, device="cuda")
    wide[..., :64], wide[..., 64:128], wide[..., 128:] = q.cuda(), k.cuda(), v.cuda()
    out_wide = torch.full((N, L, H, 2 * M), float("nan"), device="cuda")
    lengths = torch.tensor([300, 123])
    fused(lib, wide[..., :64], wide[..., 64:128], wide[..., 128:], lengths.cuda(), 0.25,
          out=out_wide[..., M:])
    assert torch.isnan(out_wide[..., :M]).all()
    gate(out_wide[..., M:].cpu(), q, k, v, lengths, 0.25)


def test_constant_values_come_back_and_masked_keys_do_not_matter(lib):
    N, L, H, E, M = 2, 5000, 4, 64, 64
    q, k, _ = inputs(N, L, H, E, M, seed=8)
    v = torch.full((N, L, H, M), -3.25)
    lengths = torch.tensor([5000, 1234]).cuda()
    got = fused(lib, q.cuda(), k.cuda(), v.cuda(), lengths, 0.0)
    assert (got + 3.25).abs().max().item() < 1e-4
    # keys and values beyond the length are never seen
    k2, v2 = k.clone(), torch.randn(N, L, H, M, generator=torch.Generator().manual_seed(9))
    v3 = v2.clone()
    k2[1, 1234:] = 50.0
    v3[1, 1234:] = 1e6
    a = fused(lib, q.cuda(), k.cuda(), v2.cuda(), lengths, 1e-6)
    b = fused(lib, q.cuda(), k2.cuda(), v3.cuda(), lengths, 1e-6)
    assert torch.equal(a, b)


def test_prefix_property_at_full_size(lib):
    """Config 4's operator shape: the first rows of a long call equal a short call's rows to
    rounding (the segmentation differs), and a repeated call is bit-identical."""
    N, L, H, E, M = 10, 4096, 8, 64, 64
    q, k, v = (t.cuda() for t in inputs(N, L, H, E, M, seed=4))
    whole = fused(lib, q, k, v, None, 1e-6)
    again = fused(lib, q, k, v, None, 1e-6)
    assert torch.equal(whole, again)
    short = fused(lib, q[:, :1500].contiguous(), k[:, :1500].contiguous(),
                  v[:, :1500].contiguous(), None, 1e-6)
    assert scale_error(whole[:, :1500].permute(0, 2, 1, 3), short.permute(0, 2, 1, 3)) <= 2e-6
    # a bounded sample against the CPU restatement
    got = whole[:2].cpu()
    gate(got, q[:2].cpu(), k[:2].cpu(), v[:2].cpu(), None, 1e-6)


def test_sizes_without_a_fused_kernel_are_refused(lib):
    from fast_transformers_amd import _native
    assert lib.ftc_causal_linear_attention_workspace_bytes(1, 1, 64, 48, 64, _native.FTC_F32) == -2
    assert lib.ftc_causal_linear_attention_workspace_bytes(1, 1, 64, 64, 64, _native.FTC_BF16) == -2
    q = torch.zeros(1, 64, 1, 48, device="cuda")
    v = torch.zeros(1, 64, 1, 64, device="cuda")
    d = [_native.describe(t.permute(0, 2, 1, 3)) for t in (q, q, v, v.clone())]
    rc = lib.ftc_causal_linear_attention(ctypes.byref(d[0]), ctypes.byref(d[1]), ctypes.byref(d[2]),
                                         None, ctypes.c_float(1e-6), ctypes.byref(d[3]), None, 0,
                                         None)
    assert rc == -2 and "fused" in _native.last_error()


def _count_backward_calls():
    """Context that counts the calls of the fused backward (autograd runs it on a thread of its
    own, where ftc_last_kernel() of this thread does not see it)."""
    import contextlib
    from fast_transformers_amd import causal_product as cpm

    @contextlib.contextmanager
    def counting():
        calls = []
        native = cpm.causal_linear_attention_backward_hip
        cpm.causal_linear_attention_backward_hip = lambda *a: (calls.append(1), native(*a))[1]
        try:
            yield calls
        finally:
            cpm.causal_linear_attention_backward_hip = native
    return counting()


def _composition(cla):
    """Context that makes the module compose its result from operator calls (what sizes and
    feature maps without a fused kernel get)."""
    import contextlib

    @contextlib.contextmanager
    def off():
        covers = cla.fused_attention_covers
        cla.fused_attention_covers = lambda *a: False
        try:
            yield
        finally:
            cla.fused_attention_covers = covers
    return off()


def test_module_takes_the_fused_path_and_agrees_with_the_composition(lib):
    from fast_transformers_amd import attention, masking
    from fast_transformers_amd.attention import causal_linear_attention as cla
    N, L, H, E, M = 2, 700, 4, 64, 64
    q, k, v = (t.cuda() for t in inputs(N, L, H, E, M, seed=11))
    lengths = masking.LengthMask(torch.tensor([700, 301]).cuda(), max_len=L)
    full = masking.LengthMask(torch.full((N,), L).cuda(), max_len=L)
    mask = masking.TriangularCausalMask(L, device="cuda")
    module = attention.CausalLinearAttention(E).cuda()
    calls = []
    native = cla.causal_linear_attention_hip
    cla.causal_linear_attention_hip = lambda *a: (calls.append(1), native(*a))[1]
    try:
        with torch.no_grad():
            y_fused = module(q, k, v, mask, full, lengths)
        assert calls == [1]
        with _composition(cla):
            y_composed = module(q.clone().requires_grad_(True), k, v, mask, full, lengths)
        assert calls == [1] and y_composed.requires_grad
    finally:
        cla.causal_linear_attention_hip = native
    assert scale_error(y_fused.permute(0, 2, 1, 3), y_composed.detach().permute(0, 2, 1, 3)) <= 1e-5
    gate(y_fused.cpu(), q.cpu(), k.cpu(), v.cpu(), torch.tensor([700, 301]), module.eps)


def _dense_attention(q, k, v, lengths, eps):
    """The closed form of the reference's API test (tests/causal_product/test_causal_product.py:
    34-40) with the feature map and the key-length mask of the module, on (N, L, H, X) tensors
    of any float type: differentiable, so that autograd gives the gradients to compare with."""
    Q = torch.nn.functional.elu(q) + 1
    K = torch.nn.functional.elu(k) + 1
    L = q.shape[1]
    keep = (torch.arange(L, device=q.device)[None, :] < lengths[:, None]).to(q.dtype)
    K = K * keep[:, :, None, None]
    QK = torch.einsum("nlhe,nshe->nhls", Q, K)
    QK = QK * torch.tril(torch.ones(L, L, dtype=q.dtype, device=q.device))
    Z = 1 / (QK.sum(dim=-1) + eps)                       # (N, H, L)
    return torch.einsum("nhls,nshm->nlhm", QK, v) * Z.permute(0, 2, 1)[..., None]


BACKWARD_SHAPES = [
    # N, L, H, E, M, key lengths
    (2, 300, 3, 64, 64, [300, 117]), (1, 1000, 8, 64, 64, [1000]), (3, 257, 2, 32, 32, [257, 40, 200]),
    (2, 513, 2, 64, 32, [513, 400]), (2, 200, 4, 32, 64, [0, 200]), (1, 33, 1, 64, 64, [33]),
]


@pytest.mark.parametrize("shape", BACKWARD_SHAPES, ids=lambda s: "n%d_l%d_h%d_e%d_m%d" % s[:5])
def test_backward_against_autograd_in_float64(lib, shape):
    """ftc_causal_linear_attention_backward (through the autograd Function the module uses)
    against autograd through the dense closed form in float64; the same closed form in
    float32 shows what that arithmetic alone costs."""
    from fast_transformers_amd.causal_product import CausalLinearAttentionFunction
    N, L, H, E, M, lens = shape
    q, k, v = inputs(N, L, H, E, M, seed=31 + L)
    g = torch.randn(N, L, H, M, generator=torch.Generator().manual_seed(32 + L))
    lengths = torch.tensor(lens)
    eps = 1e-6

    def grads(dtype, device):
        qq, kk, vv = (t.to(device=device, dtype=dtype).requires_grad_(True) for t in (q, k, v))
        out = _dense_attention(qq, kk, vv, lengths.to(device), eps)
        out.backward(g.to(device=device, dtype=dtype))
        return [out.detach().cpu()] + [t.grad.cpu() for t in (qq, kk, vv)]

    exact = grads(torch.float64, "cpu")
    plain = grads(torch.float32, "cuda")
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    nlh = lambda t: t.permute(0, 2, 1, 3)
    out = CausalLinearAttentionFunction.apply(nlh(qd), nlh(kd), nlh(vd), lengths.cuda(), eps)
    assert lib.ftc_last_kernel().startswith(b"scan_wg_kernel")
    with _count_backward_calls() as calls:
        nlh(out).backward(g.cuda())
    assert calls == [1]
    torch.cuda.synchronize()
    got = [nlh(out).detach().cpu()] + [t.grad.cpu() for t in (qd, kd, vd)]
    for name, a, b, c in zip(("out", "grad_queries", "grad_keys", "grad_values"), got, plain, exact):
        assert torch.isfinite(a).all(), name
        nlhx = lambda t: t.permute(0, 2, 1, 3).double()
        e_hip, e_plain = scale_error(nlhx(a), nlhx(c)), scale_error(nlhx(b), nlhx(c))
        print("%-13s vs float64: hip %.3e  dense fp32 autograd %.3e" % (name, e_hip, e_plain), flush=True)
        assert e_hip <= max(4 * e_plain, 5e-6), name
    # keys at or beyond the key length have no gradient, as in the reference (their features
    # are multiplied by zero)
    for n_, len_ in enumerate(lens):
        assert (got[2][n_, len_:] == 0).all()


def test_backward_finite_differences(lib):
    """Directional derivatives of sum(out * w) along random directions, by central differences
    of the float64 closed form, against the fused backward's gradients."""
    from fast_transformers_amd.causal_product import CausalLinearAttentionFunction
    N, L, H, E, M = 1, 150, 2, 64, 64
    q, k, v = inputs(N, L, H, E, M, seed=41)
    w = torch.randn(N, L, H, M, generator=torch.Generator().manual_seed(42))
    lengths = torch.tensor([131])
    eps = 1e-6
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    nlh = lambda t: t.permute(0, 2, 1, 3)
    out = CausalLinearAttentionFunction.apply(nlh(qd), nlh(kd), nlh(vd), lengths.cuda(), eps)
    (nlh(out) * w.cuda()).sum().backward()
    f = lambda a, b, c: (_dense_attention(a.double(), b.double(), c.double(), lengths, eps) * w.double()).sum()
    gen = torch.Generator().manual_seed(43)
    for name, base, grad in (("queries", 0, qd.grad), ("keys", 1, kd.grad), ("values", 2, vd.grad)):
        for _ in range(3):
            args = [q, k, v]
            direction = torch.randn(args[base].shape, generator=gen)
            h = 1e-4
            plus, minus = list(args), list(args)
            plus[base] = args[base].double() + h * direction.double()
            minus[base] = args[base].double() - h * direction.double()
            fd = ((f(*plus) - f(*minus)) / (2 * h)).item()
            an = (grad.cpu().double() * direction.double()).sum().item()
            print("d/d%s: finite difference %.6e, backward %.6e" % (name, fd, an), flush=True)
            assert abs(fd - an) <= 1e-4 * max(1.0, abs(fd))


def test_module_trains_through_the_fused_backward(lib):
    """Under grad the module runs the fused forward and its backward, and the parameters'
    gradients agree with those of the composition of operator calls."""
    from fast_transformers_amd import attention, masking
    from fast_transformers_amd.attention import causal_linear_attention as cla
    N, L, H, E, M = 2, 400, 4, 64, 64
    q, k, v = (t.cuda() for t in inputs(N, L, H, E, M, seed=51))
    lengths = masking.LengthMask(torch.tensor([400, 255]).cuda(), max_len=L)
    full = masking.LengthMask(torch.full((N,), L).cuda(), max_len=L)
    mask = masking.TriangularCausalMask(L, device="cuda")
    module = attention.CausalLinearAttention(E).cuda()
    w = torch.randn(N, L, H, M, generator=torch.Generator().manual_seed(52)).cuda()

    def run():
        leaves = [t.clone().requires_grad_(True) for t in (q, k, v)]
        y = module(*leaves, mask, full, lengths)
        (y * w).sum().backward()
        return y.detach(), [t.grad for t in leaves]

    with _count_backward_calls() as calls:
        y_fused, g_fused = run()
        assert calls == [1]
        with _composition(cla):
            y_comp, g_comp = run()
        assert calls == [1]
    nlh = lambda t: t.permute(0, 2, 1, 3)
    assert scale_error(nlh(y_fused), nlh(y_comp)) <= 1e-5
    for name, a, b in zip(("queries", "keys", "values"), g_fused, g_comp):
        err = scale_error(nlh(a), nlh(b))
        print("grad %s: fused against composition %.3e" % (name, err), flush=True)
        assert err <= 2e-5, name


def test_non_finite_inputs_propagate_as_in_the_composition(lib):
    """The feature map elu(x) + 1 keeps NaN (and maps -inf to 0, +inf to +inf), in the fused
    launch as in the composition of operator calls that training uses: the same rows come out
    non-finite either way."""
    from fast_transformers_amd import attention, masking
    N, L, H, E, M = 1, 300, 2, 64, 64
    q, k, v = (t.cuda() for t in inputs(N, L, H, E, M, seed=12))
    q[0, 40, 0, 3] = float("nan")     # one query row of head 0
    k[0, 200, 1, 5] = float("nan")    # a key of head 1: every row from 200 on
    q[0, 10, 1, 7] = float("-inf")    # phi(-inf) = 0: harmless
    full = masking.LengthMask(torch.full((N,), L).cuda(), max_len=L)
    mask = masking.TriangularCausalMask(L, device="cuda")
    module = attention.CausalLinearAttention(E).cuda()
    with torch.no_grad():
        y_fused = module(q, k, v, mask, full, full)
    y_composed = module(q.clone().requires_grad_(True), k, v, mask, full, full).detach()
    bad_fused, bad_composed = ~torch.isfinite(y_fused), ~torch.isfinite(y_composed)
    assert torch.equal(bad_fused.any(dim=-1), bad_composed.any(dim=-1))
    assert bad_fused[0, 40, 0].all() and bad_fused[0, 200:, 1].all()
    assert not bad_fused[0, :40, 0].any() and not bad_fused[0, :200, 1].any()
    ok = ~bad_fused
    assert (y_fused[ok] - y_composed[ok]).abs().max() <= 1e-4 * y_composed[ok].abs().max()


def test_forward_and_backward_replay_in_a_graph(lib):
    """Both entry points only enqueue kernels (fill kernels instead of memsets, nothing
    allocated), so a forward + backward pair can be captured in a HIP graph.  Every replay,
    with direct launches on other data in between, reproduces the direct results bit for bit."""
    from fast_transformers_amd import causal_product as cp
    N, L, H, E, M = 2, 600, 4, 64, 64
    nlh = lambda t: t.permute(0, 2, 1, 3)
    q, k, v = (nlh(t.cuda()) for t in inputs(N, L, H, E, M, seed=71))
    q2, k2, v2 = (nlh(t.cuda()) for t in inputs(N, L, H, E, M, seed=72))
    g = nlh(torch.randn(N, L, H, M, generator=torch.Generator().manual_seed(73)).cuda())
    lengths = torch.tensor([600, 431]).cuda()
    out = nlh(torch.empty(N, L, H, M, device="cuda"))
    den = torch.empty(N, H, L, device="cuda")
    grads = [nlh(torch.empty(N, L, H, X, device="cuda")) for X in (E, E, M)]

    def pair():
        cp.causal_linear_attention_hip(q, k, v, lengths, 1e-6, out, den)
        cp.causal_linear_attention_backward_hip(q, k, v, lengths, out, den, g, *grads)

    pair()
    torch.cuda.synchronize()
    want = [t.clone() for t in [out] + grads]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # the wrapper's workspace for this stream exists before capture
        pair()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        pair()
    other = nlh(torch.empty(N, L, H, M, device="cuda"))
    for replay in range(4):
        for t in [out, den] + grads:
            t.fill_(float("nan"))
        cp.causal_linear_attention_hip(q2, k2, v2, None, 1e-6, other)   # the program's own work
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("out", "dq", "dk", "dv"), [out] + grads, want):
            assert torch.equal(got, ref), (replay, name)
    assert torch.isfinite(other).all()
