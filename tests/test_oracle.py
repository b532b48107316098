"""Pins the CPU checker (oracle/) before anything is compared against it.

Checks, each chosen so that a plausible mistake fails it:
  * the reference's own compiled CPU extension (oracle/_ref, when built): bit-exact;
  * the golden vectors that extension wrote (tests/golden/*.npz);
  * the dense closed form tril(Q K^T) V and its gradients in float64, with the metric
    and bound of the reference's tests (test_causal_product_cpu.py:19-20,49,72-74);
  * brute-force triple loops on tiny inputs (inclusive diagonal, operand order);
  * special cases: E = 1 is a cumulative sum; causality; the prefix property;
    time reversal links the forward product to the dK/dV passes.
"""
import glob
import os

import numpy as np
import pytest
import torch

import oracle


def max_relative_error(a, b, eps=1e-6):
    # tests/causal_product/test_causal_product_cpu.py:19-20
    return torch.abs((a - b) / (torch.abs(a) + eps)).max().item()


SHAPES = [(2, 3, 50, 17, 33), (1, 2, 100, 64, 64), (1, 1, 64, 130, 10), (3, 1, 7, 1, 1)]


@pytest.mark.skipif(not oracle.reference_extension_available(), reason="oracle/_ref not built")
@pytest.mark.parametrize("shape", SHAPES)
def test_restatement_is_bit_exact_with_reference_extension(shape):
    ref = oracle.load_reference_extension()
    N, H, L, E, M = shape
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=sum(shape))
    out_ref = torch.zeros(N, H, L, M)
    ref.causal_dot_product(Q, K, V, out_ref)
    assert torch.equal(oracle.forward(Q, K, V), out_ref)
    g_ref = [torch.zeros_like(x) for x in (Q, K, V)]
    ref.causal_dot_backward(Q, K, V, G, *g_ref)
    for a, b in zip(oracle.backward(Q, K, V, G), g_ref):
        assert torch.equal(a, b)


@pytest.mark.skipif(not oracle.reference_extension_available(), reason="oracle/_ref not built")
def test_restatement_matches_reference_extension_on_strided_views():
    ref = oracle.load_reference_extension()
    N, H, L, E, M = 2, 3, 40, 20, 24
    gen = torch.Generator().manual_seed(5)
    # (N, L, H, X) storage viewed as (N, H, L, X): what a caller gets from permute()
    Q = torch.rand(N, L, H, E, generator=gen).permute(0, 2, 1, 3)
    K = torch.rand(N, L, H, E, generator=gen).permute(0, 2, 1, 3)
    V = torch.randn(N, L, H, M, generator=gen).permute(0, 2, 1, 3)
    G = torch.randn(N, L, H, M, generator=gen).permute(0, 2, 1, 3)
    out_ref = torch.zeros(N, H, L, M)
    ref.causal_dot_product(Q, K, V, out_ref)
    out = torch.full((N, L, H, M), float("nan")).permute(0, 2, 1, 3)
    oracle.causal_dot_product(Q, K, V, out)
    assert torch.equal(out, out_ref)
    g_ref = [torch.zeros(N, H, L, X) for X in (E, E, M)]
    ref.causal_dot_backward(Q, K, V, G, *g_ref)
    g = [torch.full((N, H, L, X), float("nan")) for X in (E, E, M)]
    oracle.causal_dot_backward(Q, K, V, G, *g)
    for a, b in zip(g, g_ref):
        assert torch.equal(a, b)


def _golden_files():
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    return sorted(glob.glob(os.path.join(here, "causal_*.npz")))


def test_golden_vectors_exist():
    assert len(_golden_files()) >= 6


@pytest.mark.parametrize("path", _golden_files(), ids=os.path.basename)
def test_restatement_reproduces_golden_vectors(path):
    z = np.load(path)
    Q, K, V, G = (torch.from_numpy(z[k]) for k in "QKVG")
    out = oracle.forward(Q, K, V)
    dQ, dK, dV = oracle.backward(Q, K, V, G)
    for got, key in ((out, "product"), (dQ, "grad_queries"), (dK, "grad_keys"),
                     (dV, "grad_values")):
        want = torch.from_numpy(z[key])
        scale = want.abs().max().item()
        assert (got - want).abs().max().item() <= 1e-6 * scale, key


@pytest.mark.parametrize("path", _golden_files(), ids=os.path.basename)
def test_golden_vectors_satisfy_dense_closed_form(path):
    """The stored reference outputs themselves obey tril(Q K^T) V in float64."""
    z = np.load(path)
    Q, K, V, G = (torch.from_numpy(z[k]).double() for k in "QKVG")
    want = (oracle.dense_forward(Q, K, V),) + oracle.dense_backward(Q, K, V, G)
    for w, key in zip(want, ("product", "grad_queries", "grad_keys", "grad_values")):
        got = torch.from_numpy(z[key]).double()
        assert (got - w).abs().max().item() <= 2e-6 * w.abs().max().item(), key


@pytest.mark.parametrize("trial", range(4))
def test_forward_against_dense_form_reference_protocol(trial):
    # test_causal_product_cpu.py:32-49 with seeded draws and a smaller batch
    rng = np.random.RandomState(100 + trial)
    N, H, L = 3, 4, 100
    E, M = int(rng.randint(10, 256)), int(rng.randint(10, 256))
    Q, K, V, _ = oracle.make_inputs(N, H, L, E, M, seed=trial, positive_uniform=True)
    out = oracle.forward(Q, K, V)
    dense = oracle.dense_forward(Q.double(), K.double(), V.double()).float()
    assert max_relative_error(dense, out) < 1e-5


@pytest.mark.parametrize("trial", range(4))
def test_backward_against_autograd_of_dense_form(trial):
    # test_causal_product_cpu.py:51-74
    rng = np.random.RandomState(200 + trial)
    N, H, L = 2, 3, 100
    E, M = int(rng.randint(10, 256)), int(rng.randint(10, 256))
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=50 + trial, positive_uniform=True)
    dQ, dK, dV = oracle.backward(Q, K, V, G)
    Qd, Kd, Vd = (x.double().requires_grad_(True) for x in (Q, K, V))
    out = oracle.dense_forward(Qd, Kd, Vd)
    torch.einsum("nhlm,nhlm->", out, G.double()).backward()
    assert max_relative_error(Qd.grad.float(), dQ) < 1e-5
    assert max_relative_error(Kd.grad.float(), dK) < 1e-5
    assert max_relative_error(Vd.grad.float(), dV) < 1e-5
    # and the written-out gradient formulas agree with autograd
    for a, b in zip(oracle.dense_backward(Q.double(), K.double(), V.double(), G.double()),
                    (Qd.grad, Kd.grad, Vd.grad)):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_float64_build_gradients_by_finite_differences():
    N, H, L, E, M = 1, 1, 6, 3, 4
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=9, dtype=torch.float64)
    dQ, dK, dV = oracle.backward(Q, K, V, G)

    def loss(q, k, v):
        return (oracle.forward(q, k, v) * G).sum().item()

    eps = 1e-6
    for x, dx, which in ((Q, dQ, 0), (K, dK, 1), (V, dV, 2)):
        for idx in [(0, 0, 0, 0), (0, 0, 2, 1), (0, 0, L - 1, x.shape[3] - 1)]:
            xp, xm = x.clone(), x.clone()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = [Q, K, V]
            args_m = [Q, K, V]
            args_p[which], args_m[which] = xp, xm
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - dx[idx].item()) < 1e-6 * max(1.0, abs(fd))


def test_brute_force_tiny():
    N, H, L, E, M = 1, 2, 5, 3, 2
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=3, dtype=torch.float64)
    out = oracle.forward(Q, K, V)
    dQ, dK, dV = oracle.backward(Q, K, V, G)
    want = torch.zeros(N, H, L, M, dtype=torch.float64)
    wq, wk, wv = torch.zeros_like(Q), torch.zeros_like(K), torch.zeros_like(V)
    for h in range(H):
        for l in range(L):
            for j in range(l + 1):  # inclusive: position l sees key l
                qk = sum(Q[0, h, l, e] * K[0, h, j, e] for e in range(E))
                gv = sum(G[0, h, l, m] * V[0, h, j, m] for m in range(M))
                for m in range(M):
                    want[0, h, l, m] += qk * V[0, h, j, m]
                    wv[0, h, j, m] += qk * G[0, h, l, m]
                for e in range(E):
                    wq[0, h, l, e] += gv * K[0, h, j, e]
                    wk[0, h, j, e] += gv * Q[0, h, l, e]
    for a, b in ((out, want), (dQ, wq), (dK, wk), (dV, wv)):
        assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_first_position_and_unit_width():
    Q, K, V, _ = oracle.make_inputs(2, 2, 9, 1, 5, seed=4, dtype=torch.float64)
    out = oracle.forward(Q, K, V)
    # E = 1: out_l = q_l * cumsum_l(k v)
    want = Q * torch.cumsum(K * V, dim=2)
    assert torch.allclose(out, want, rtol=1e-12, atol=1e-12)
    Q, K, V, _ = oracle.make_inputs(1, 1, 4, 6, 3, seed=5, dtype=torch.float64)
    out = oracle.forward(Q, K, V)
    assert torch.allclose(out[0, 0, 0], (Q[0, 0, 0] @ K[0, 0, 0]) * V[0, 0, 0])
    # Q = 1: out = cumsum over L of (sum_e k_e) v
    ones = torch.ones_like(Q)
    want = torch.cumsum(K.sum(-1, keepdim=True) * V, dim=2)
    assert torch.allclose(oracle.forward(ones, K, V), want, rtol=1e-12, atol=1e-12)


def test_causality_and_prefix_property():
    N, H, L, E, M = 1, 2, 40, 8, 8
    Q, K, V, _ = oracle.make_inputs(N, H, L, E, M, seed=6)
    out = oracle.forward(Q, K, V)
    K2, V2 = K.clone(), V.clone()
    K2[:, :, 25] += 1.0
    V2[:, :, 25] -= 2.0
    out2 = oracle.forward(Q, K2, V2)
    assert torch.equal(out[:, :, :25], out2[:, :, :25])
    assert not torch.equal(out[:, :, 25], out2[:, :, 25])
    short = oracle.forward(Q[:, :, :17].contiguous(), K[:, :, :17].contiguous(),
                           V[:, :, :17].contiguous())
    assert torch.equal(short, out[:, :, :17])


def test_role_and_time_reversal_identities():
    """dQ = fwd(G, V, K); dK = flip(fwd(flip V, flip G, flip Q)); dV = flip(fwd(flip K, flip Q, flip G))."""
    Q, K, V, G = oracle.make_inputs(1, 2, 30, 5, 7, seed=7, dtype=torch.float64)
    dQ, dK, dV = oracle.backward(Q, K, V, G)
    flip = lambda t: torch.flip(t, dims=[2]).contiguous()
    assert torch.allclose(dQ, oracle.forward(G, V, K), rtol=1e-12, atol=1e-12)
    assert torch.allclose(dK, flip(oracle.forward(flip(V), flip(G), flip(Q))), rtol=1e-12,
                          atol=1e-12)
    assert torch.allclose(dV, flip(oracle.forward(flip(K), flip(Q), flip(G))), rtol=1e-12,
                          atol=1e-12)


def test_recurrent_form_agrees():
    # tests/recurrent/attention/self_attention/test_linear_attention.py:54-79 (1e-5 abs)
    Q, K, V, _ = oracle.make_inputs(2, 2, 60, 25, 64, seed=8, positive_uniform=True)
    out = oracle.forward(Q, K, V)
    rec = oracle.recurrent_forward(Q.double(), K.double(), V.double())
    assert (out.double() - rec).abs().max().item() < 1e-5 * max(1.0, rec.abs().max().item())


def test_outputs_need_not_be_zeroed():
    Q, K, V, G = oracle.make_inputs(1, 1, 10, 4, 4, seed=10)
    out = torch.full((1, 1, 10, 4), 7.0)
    oracle.causal_dot_product(Q, K, V, out)
    assert torch.equal(out, oracle.forward(Q, K, V))


# ---------------------------------------------------------------------------
# the forward with the running state handed in and out
# ---------------------------------------------------------------------------
def test_stateful_forward_from_zero_is_the_forward_and_ends_on_kt_v():
    Q, K, V, _ = oracle.make_inputs(2, 3, 70, 9, 6, seed=41)
    out, state = oracle.forward_with_state(Q, K, V)
    assert torch.equal(out, oracle.forward(Q, K, V))
    exact = torch.einsum("nhle,nhlm->nhem", K.double(), V.double())
    # V has zero mean, so single entries cancel; the yardstick is the size of the state
    assert (state.double() - exact).abs().max() / exact.abs().max() < 1e-6


def test_stateful_forward_hands_the_state_over_between_pieces():
    """Two pieces with the state passed on are one pass: the running state after position
    l is the same sequence of operations either way, so the match is exact."""
    Q, K, V, _ = oracle.make_inputs(2, 2, 90, 7, 5, seed=42)
    whole, end = oracle.forward_with_state(Q, K, V)
    for cut in (1, 33, 89):
        o1, s1 = oracle.forward_with_state(Q[:, :, :cut], K[:, :, :cut], V[:, :, :cut])
        o2, s2 = oracle.forward_with_state(Q[:, :, cut:], K[:, :, cut:], V[:, :, cut:], s1)
        assert torch.equal(torch.cat([o1, o2], dim=2), whole)
        assert torch.equal(s2, end)


def test_stateful_forward_initial_state_adds_q_times_state():
    Q, K, V, _ = oracle.make_inputs(1, 3, 40, 6, 8, seed=43, dtype=torch.float64)
    s0 = torch.randn(1, 3, 6, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(7))
    out, end = oracle.forward_with_state(Q, K, V, s0)
    want = oracle.dense_forward(Q, K, V) + torch.einsum("nhle,nhem->nhlm", Q, s0)
    assert max_relative_error(out, want) < 1e-12
    assert max_relative_error(end, s0 + torch.einsum("nhle,nhlm->nhem", K, V)) < 1e-12


def test_stateful_forward_continues_into_the_stepwise_form():
    """The final state is the Si of the reference's step-wise module
    (recurrent/attention/self_attention/linear_attention.py:79-88): stepping on from it with
    the einsum form gives the rows the batched pass gives."""
    Q, K, V, _ = oracle.make_inputs(2, 2, 30, 5, 4, seed=44, dtype=torch.float64)
    cut = 21
    _, S = oracle.forward_with_state(Q[:, :, :cut], K[:, :, :cut], V[:, :, :cut])
    whole = oracle.forward(Q, K, V)
    for l in range(cut, 30):
        S = S + torch.einsum("nhd,nhm->nhdm", K[:, :, l], V[:, :, l])
        row = torch.einsum("nhd,nhdm->nhm", Q[:, :, l], S)
        assert max_relative_error(row, whole[:, :, l]) < 1e-12


# ---------------------------------------------------------------------------
# the caller restated: feature map, key-length mask, normaliser
# ---------------------------------------------------------------------------
def _attention_inputs(N, L, H, E, M, seed, dtype=torch.float64):
    gen = torch.Generator().manual_seed(seed)
    q = 1.5 * torch.randn(N, L, H, E, generator=gen)
    k = 1.5 * torch.randn(N, L, H, E, generator=gen)
    v = torch.randn(N, L, H, M, generator=gen)
    return q.to(dtype), k.to(dtype), v.to(dtype)


def test_attention_restatement_reproduces_the_reference_module_outputs():
    """tests/golden/attention_causal_linear.npz holds what the reference's own
    CausalLinearAttention returned (make_encoder_golden.py)."""
    import numpy as np
    import os
    data = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_causal_linear.npz"))
    for tag in ("a", "b"):
        q, k, v, y = (torch.from_numpy(data[tag + "_" + x]) for x in ("q", "k", "v", "y"))
        lengths = torch.from_numpy(data[tag + "_lengths"])
        got = oracle.causal_linear_attention(q, k, v, lengths, float(data[tag + "_eps"]))
        assert got.shape == y.shape
        assert (got - y).abs().max().item() < 1e-5 * max(1.0, y.abs().max().item())
        # the ragged entry really is ragged: it differs from the unmasked result past its length
        full = oracle.causal_linear_attention(q, k, v, None, float(data[tag + "_eps"]))
        n, cut = 1, int(lengths[1])
        assert torch.equal(full[n, :cut], got[n, :cut])
        assert (full[n, cut:] - got[n, cut:]).abs().max() > 1e-3


def test_attention_restatement_is_the_dense_normalised_form():
    """tests/causal_product/test_causal_product.py:34-40: masked phi(Q) phi(K)^T, rows divided
    by their sums (+ eps), times V."""
    q, k, v = _attention_inputs(2, 45, 3, 6, 5, seed=51)
    lengths = torch.tensor([45, 17])
    got = oracle.causal_linear_attention(q, k, v, lengths, eps=1e-6)
    phi = lambda x: torch.where(x > 0, x + 1, torch.exp(x))
    keep = (torch.arange(45)[None, :] < lengths[:, None]).double()
    A = torch.einsum("nlhe,nshe->nhls", phi(q), phi(k) * keep[:, :, None, None])
    A = A * torch.tril(torch.ones(45, 45, dtype=torch.float64))
    A = A / (A.sum(-1, keepdim=True) + 1e-6)
    want = torch.einsum("nhls,nshm->nlhm", A, v)
    assert max_relative_error(got, want) < 1e-9


def test_attention_restatement_is_the_stepwise_form():
    """recurrent/attention/self_attention/linear_attention.py:55-88: Zi += phi(k);
    Si += phi(k) v^T; out = phi(q) Si / (phi(q) . Zi + eps)."""
    q, k, v = _attention_inputs(2, 33, 2, 4, 7, seed=52)
    got = oracle.causal_linear_attention(q, k, v, None, eps=1e-6)
    phi = lambda x: torch.nn.functional.elu(x) + 1
    Si = torch.zeros(2, 2, 4, 7, dtype=torch.float64)
    Zi = torch.zeros(2, 2, 4, dtype=torch.float64)
    for l in range(33):
        Q, K = phi(q[:, l]), phi(k[:, l])
        Zi = Zi + K
        Si = Si + torch.einsum("nhd,nhm->nhdm", K, v[:, l])
        Z = 1. / (torch.einsum("nhd,nhd->nh", Q, Zi) + 1e-6)
        V = torch.einsum("nhd,nhdm,nh->nhm", Q, Si, Z)
        assert max_relative_error(got[:, l], V) < 1e-9


def test_attention_rows_are_convex_combinations_of_values():
    """With eps = 0 every output row is a weighted mean of the values seen so far (weights
    positive, summing to one): constant values come back unchanged."""
    q, k, _ = _attention_inputs(1, 50, 2, 8, 3, seed=53)
    v = torch.full((1, 50, 2, 3), 2.5, dtype=torch.float64)
    got = oracle.causal_linear_attention(q, k, v, None, eps=0.0)
    assert (got - 2.5).abs().max().item() < 1e-9
