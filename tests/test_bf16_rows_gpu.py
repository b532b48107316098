"""bf16 rows on the chain-parallel kernel's fp16 path (its form that takes rows of either
element type, scan by scan): the three scans of a backward call over up to 128 chains, a
forward over at least 256 chains, and widths that the other matrix-core kernels would only
take as padded copies.

bf16 values are exact in one fp16 piece after scaling, so the arithmetic is that of fp32 rows
whose low pieces are zero: the fp32 product must be as close to float64 as the CPU checker's
(on the same bf16-rounded inputs), and a bf16 gradient must be the float64 gradient rounded to
bf16, give or take one unit in the last place where the fp32 value lies near a rounding
boundary."""
import pytest
import torch

import oracle
from parity import scale_error

pytestmark = pytest.mark.gpu

KERNELS = (b"scan_tph_kernel", b"scan_tph_kernel (exchange)")


@pytest.fixture(scope="module")
def cp():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU (torch.cuda.is_available() is False)")
    from fast_transformers_amd import causal_product
    from fast_transformers_amd import _native
    _native.load()
    return causal_product


def _last_kernel():
    from fast_transformers_amd import _native
    return _native.load().ftc_last_kernel()


def _inputs(N, H, L, E, M, seed):
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=seed)
    return Q.bfloat16(), K.bfloat16(), V.bfloat16(), G


def _bf16_ulps(got, exact):
    """Largest distance, in bf16 units in the last place of the exact value, between a bf16
    result and the float64 value it stands for."""
    exact = exact.double()
    ulp = torch.exp2(torch.floor(torch.log2(exact.abs().clamp_min(1e-30))) - 7)
    return ((got.double() - exact).abs() / ulp).max().item()


def _check_gradients(tag, grads, Qb, Kb, Vb, G):
    exact = oracle.backward(Qb.double(), Kb.double(), Vb.double(), G.double())
    refs = oracle.backward(Qb.float(), Kb.float(), Vb.float(), G)
    for key, got, want, ref in zip(("dQ", "dK", "dV"), grads, exact, refs):
        assert got.dtype == torch.bfloat16, key
        got = got.float().cpu()
        assert torch.isfinite(got).all(), key
        s = scale_error(got, ref)
        # half a unit from the rounding to bf16, plus what the fp32 sums are away from float64:
        # never a whole unit more, except for values that cancel to far below the row's scale
        big = want.abs() >= 2.0 ** -6 * want.abs().amax(dim=-1, keepdim=True)
        u = _bf16_ulps(got[big], want[big])
        print("%-30s %s: scale error vs fp32 checker %.3e, worst distance %.2f bf16 ulp" %
              (tag, key, s, u), flush=True)
        assert s <= 2 ** -8, key
        assert u <= 1.0, key


BACKWARD_SHAPES = {
    # name: (N, H, L, E, M, seed)
    "headline_shape": (10, 8, 1000, 64, 64, 31),
    "short_chains": (6, 8, 300, 64, 64, 32),
    "rows_of_48_and_40": (6, 8, 257, 48, 40, 33),       # no padded copies: clipped widths
    "state_of_32_rows": (8, 8, 520, 32, 64, 34),
    "long_chains_cut_with_an_exchange": (4, 8, 4096, 64, 64, 35),
}


@pytest.mark.parametrize("name", sorted(BACKWARD_SHAPES))
def test_backward_of_bf16_rows(cp, name):
    N, H, L, E, M, seed = BACKWARD_SHAPES[name]
    print("bf16 rows, backward", name, (N, H, L, E, M), flush=True)
    Qb, Kb, Vb, G = _inputs(N, H, L, E, M, seed)
    grads = [torch.full((N, H, L, X), float("nan"), device="cuda", dtype=torch.bfloat16)
             for X in (E, E, M)]
    cp.causal_dot_backward_hip(Qb.cuda(), Kb.cuda(), Vb.cuda(), G.cuda(), *grads)
    if E == M:  # (else dV is a launch of its own, a single scan, which stays where it was)
        assert _last_kernel() in KERNELS, _last_kernel()
    _check_gradients(name, grads, Qb, Kb, Vb, G)


FORWARD_SHAPES = {
    "256_chains": (16, 16, 200, 64, 64, 41),
    "256_chains_of_one_chunk_and_a_bit": (32, 8, 40, 64, 64, 42),
    "rows_of_48_and_40": (6, 8, 257, 48, 40, 43),
    "rows_of_20": (8, 8, 130, 20, 20, 44),
}


@pytest.mark.parametrize("name", sorted(FORWARD_SHAPES))
def test_forward_of_bf16_rows(cp, name):
    N, H, L, E, M, seed = FORWARD_SHAPES[name]
    print("bf16 rows, forward", name, (N, H, L, E, M), flush=True)
    Qb, Kb, Vb, _ = _inputs(N, H, L, E, M, seed)
    out = torch.full((N, H, L, M), float("nan"), device="cuda")
    cp.causal_dot_product_hip(Qb.cuda(), Kb.cuda(), Vb.cuda(), out)
    assert _last_kernel() in KERNELS, _last_kernel()
    ref = oracle.forward(Qb.float(), Kb.float(), Vb.float())
    exact = oracle.forward(Qb.double(), Kb.double(), Vb.double())
    e_hip, e_cpu = scale_error(out.cpu(), exact), scale_error(ref, exact)
    print("   vs float64: hip %.3e cpu %.3e" % (e_hip, e_cpu), flush=True)
    assert torch.isfinite(out).all()
    assert e_hip <= max(4 * e_cpu, 2e-6)


def test_bf16_rows_in_interleaved_heads_storage(cp):
    """(N, L, H, X) storage handed over as permuted views: rows of one chain lie H rows apart."""
    N, H, L, E, M = 6, 8, 300, 64, 64
    Qb, Kb, Vb, G = _inputs(N, H, L, E, M, 51)
    nlh = lambda t: t.permute(0, 2, 1, 3).contiguous().cuda().permute(0, 2, 1, 3)
    q, k, v, g = (nlh(t) for t in (Qb, Kb, Vb, G))
    assert not q.is_contiguous()
    grads = [torch.full((N, L, H, X), float("nan"), device="cuda", dtype=torch.bfloat16)
             .permute(0, 2, 1, 3) for X in (E, E, M)]
    cp.causal_dot_backward_hip(q, k, v, g, *grads)
    assert _last_kernel() in KERNELS, _last_kernel()
    _check_gradients("interleaved heads", grads, Qb, Kb, Vb, G)


def test_bf16_rows_far_from_one(cp):
    """Operands many orders of magnitude away from one, and values that grow along the chain
    (the running ceilings of b and v rise, the state is rescaled)."""
    N, H, L, E, M = 6, 8, 300, 64, 64
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=52)
    ramp = torch.exp2(torch.linspace(-20, 12, L))[None, None, :, None]
    Qb, Kb, Vb = (1e-3 * Q).bfloat16(), (K * ramp).bfloat16(), (3e4 * V * ramp).bfloat16()
    G = 1e-5 * G
    grads = [torch.full((N, H, L, X), float("nan"), device="cuda", dtype=torch.bfloat16)
             for X in (E, E, M)]
    cp.causal_dot_backward_hip(Qb.cuda(), Kb.cuda(), Vb.cuda(), G.cuda(), *grads)
    assert _last_kernel() in KERNELS, _last_kernel()
    exact = oracle.backward(Qb.double(), Kb.double(), Vb.double(), G.double())
    for key, got, want in zip(("dQ", "dK", "dV"), grads, exact):
        got = got.float().cpu().double()
        assert torch.isfinite(got).all(), key
        # per row: the rows differ in scale by many orders of magnitude
        num = (got - want).abs().amax(dim=-1)
        den = want.abs().amax(dim=-1)
        err = (num / den.clamp_min(1e-300))[den > 0].max().item()
        print("far from one %s: worst row error %.3e" % (key, err), flush=True)
        assert err <= 2 ** -8, key


def test_bf16_forward_with_states_handed_in_and_out(cp):
    """The stateful forward on bf16 rows: two pieces of a sequence against the whole."""
    N, H, L, E, M = 16, 16, 160, 64, 64
    Qb, Kb, Vb, _ = _inputs(N, H, L, E, M, 53)
    q, k, v = Qb.cuda(), Kb.cuda(), Vb.cuda()
    cut = 96
    first, state = cp.causal_dot_product_with_state(q[:, :, :cut], k[:, :, :cut], v[:, :, :cut])
    assert _last_kernel() in KERNELS, _last_kernel()
    second, last = cp.causal_dot_product_with_state(q[:, :, cut:], k[:, :, cut:], v[:, :, cut:], state)
    assert _last_kernel() in KERNELS, _last_kernel()
    got = torch.cat([first, second], dim=2).cpu()
    exact = oracle.forward(Qb.double(), Kb.double(), Vb.double())
    ref = oracle.forward(Qb.float(), Kb.float(), Vb.float())
    assert scale_error(got, exact) <= max(4 * scale_error(ref, exact), 2e-6)
    want_state = torch.einsum("nhle,nhlm->nhem", Kb.double(), Vb.double())
    assert scale_error(last.cpu(), want_state) <= 2e-6
