"""The caller side of the hot path: CausalLinearAttention and the encoder blocks around it.

Checked against (a) the CPU checker through the (N, L, H, X) entry without layout copies,
(b) the dense normalised masked attention the reference's API test uses
(tests/causal_product/test_causal_product.py:34-40), (c) the step-wise recurrent form the
reference tests batch attention against
(tests/recurrent/attention/self_attention/test_linear_attention.py:54-79, bound 1e-5), and
(d) the same encoder with a dense pure-torch inner attention, and (e) the outputs of a
builder-made reference encoder on its own weights (tests/golden/encoder_causal_linear.npz,
written by tests/golden/make_encoder_golden.py from the reference's modules), which pins the
block structure: projections, head split, residual and post-norm order, feed-forward, final
norm, parameter names.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from parity import scale_error

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def att():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU")
    from fast_transformers_amd import attention, masking
    attention.masking = masking
    return attention


def test_causal_linear_on_nlh_layout_matches_checker(att):
    N, L, H, E, M = 2, 333, 4, 64, 64
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed=21)          # (N, H, L, X)
    to_nlh = lambda t: t.permute(0, 2, 1, 3).contiguous()
    Qd, Kd, Vd = (to_nlh(t).cuda().requires_grad_(True) for t in (Q, K, V))
    out = att.causal_linear(Qd, Kd, Vd)
    assert out.shape == (N, L, H, M) and out.is_contiguous()
    (out * to_nlh(G).cuda()).sum().backward()
    want = oracle.forward(Q, K, V)
    refs = oracle.backward(Q, K, V, G)
    assert scale_error(out.detach().cpu().permute(0, 2, 1, 3), want) <= 1e-5
    for got, ref in zip((Qd.grad, Kd.grad, Vd.grad), refs):
        assert scale_error(got.cpu().permute(0, 2, 1, 3), ref) <= 1e-5


def _phi(x):
    """elu(x) + 1 (feature_maps/base.py:71-73)"""
    return torch.nn.functional.elu(x) + 1


def dense_attention(phi, q, k, v, key_lengths, eps):
    """phi(q) phi(k)^T masked to j <= i and to valid keys, row-normalised, times v; float64."""
    Q, K, V = phi(q.double()), phi(k.double()), v.double()
    K = K * key_lengths.float_matrix.double()[:, :, None, None]
    L = Q.shape[1]
    A = torch.einsum("nlhe,nshe->nhls", Q, K) * torch.tril(torch.ones(L, L, dtype=torch.float64,
                                                                      device=q.device))
    A = A / (A.sum(-1, keepdim=True) + eps)
    return torch.einsum("nhls,nshm->nlhm", A, V)


def test_module_against_dense_normalised_attention(att):
    m = att.masking
    N, L, H, E, M = 3, 130, 4, 32, 64
    gen = torch.Generator().manual_seed(3)
    q, k = torch.randn(N, L, H, E, generator=gen).cuda(), torch.randn(N, L, H, E, generator=gen).cuda()
    v = torch.randn(N, L, H, M, generator=gen).cuda()
    lengths = m.LengthMask(torch.tensor([L, L - 17, 40]).cuda(), max_len=L)
    layer = att.CausalLinearAttention(E)
    out = layer(q, k, v, m.TriangularCausalMask(L, device="cuda"), lengths, lengths)
    assert out.shape == (N, L, H, M) and out.is_contiguous()
    want = dense_attention(_phi, q, k, v, lengths, 1e-6)
    assert (out.double() - want).abs().max().item() < 1e-5
    with pytest.raises(RuntimeError):
        layer(q, k, v, m.FullMask(L, device="cuda"), lengths, lengths)
    # more keys than queries: sliced; fewer: zero-padded (reference :57-69)
    S = 100
    klen = m.LengthMask(torch.full((N,), S).cuda(), max_len=S)
    sliced = layer(q[:, :70], k[:, :S], v[:, :S], m.TriangularCausalMask(70, device="cuda"),
                   klen, klen)
    want70 = dense_attention(_phi, q[:, :70], k[:, :70], v[:, :70],
                             m.LengthMask(torch.full((N,), 70).cuda(), max_len=70), 1e-6)
    assert (sliced.double() - want70).abs().max().item() < 1e-5
    padded = layer(q, k[:, :S], v[:, :S], m.TriangularCausalMask(L, device="cuda"), klen, klen)
    assert padded.shape == (N, L, H, M)
    assert (padded[:, :S].double() - dense_attention(
        _phi, q[:, :S], k[:, :S], v[:, :S], klen, 1e-6)).abs().max().item() < 1e-5


def test_batch_equals_recurrent_form(att):
    """N=10, H=4, E=25, M=64, L=100, U[0,1) as in the reference test; the odd E runs on the
    shape-agnostic kernel."""
    m = att.masking
    N, L, H, E, M = 10, 100, 4, 25, 64
    gen = torch.Generator().manual_seed(4)
    q, k, v = (torch.rand(N, L, H, X, generator=gen).cuda() for X in (E, E, M))
    lengths = m.LengthMask(torch.full((N,), L).cuda(), max_len=L)
    layer = att.CausalLinearAttention(E)
    out = layer(q, k, v, m.TriangularCausalMask(L, device="cuda"), lengths, lengths)
    # recurrent form (recurrent/attention/self_attention/linear_attention.py:63-90)
    Q, K = _phi(q.double()), _phi(k.double())
    S = torch.zeros(N, H, E, M, dtype=torch.float64, device="cuda")
    Zs = torch.zeros(N, H, E, dtype=torch.float64, device="cuda")
    worst = 0.0
    for i in range(L):
        S = S + torch.einsum("nhe,nhm->nhem", K[:, i], v[:, i].double())
        Zs = Zs + K[:, i]
        Z = 1.0 / (torch.einsum("nhe,nhe->nh", Q[:, i], Zs) + 1e-6)
        step = torch.einsum("nhe,nhem,nh->nhm", Q[:, i], S, Z)
        worst = max(worst, (out[:, i].double() - step).abs().max().item())
    assert worst < 1e-5


class _DenseInner(torch.nn.Module):
    def __init__(self, eps=1e-6):
        super().__init__()
        self.eps = eps

    def forward(self, q, k, v, attn_mask, query_lengths, key_lengths):
        return dense_attention(lambda x: torch.nn.functional.elu(x) + 1, q, k, v, key_lengths,
                               self.eps).to(q.dtype)


def test_encoder_against_dense_inner_attention(att):
    m = att.masking
    torch.manual_seed(0)
    enc = att.build_causal_linear_encoder(n_layers=2, n_heads=4, query_dimensions=32,
                                          value_dimensions=32, feed_forward_dimensions=64).cuda()
    enc.eval()
    N, L = 2, 96
    x = torch.rand(N, L, 128, generator=torch.Generator().manual_seed(1)).cuda()
    mask = m.TriangularCausalMask(L, device="cuda")
    with torch.no_grad():
        y = enc(x, attn_mask=mask)
        # same weights, dense float64 inner attention
        import copy
        ref = copy.deepcopy(enc)
        for layer in ref.layers:
            layer.attention.inner_attention = _DenseInner()
        y_ref = ref(x, attn_mask=mask)
    assert y.shape == (N, L, 128)
    assert (y - y_ref).abs().max().item() < 2e-5
    # the default mask is not causal and must be refused, as in the reference
    with pytest.raises(RuntimeError):
        enc(x)
    # training step through the custom backward
    enc.train()
    out = enc(x, attn_mask=mask)
    out.sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in enc.parameters())


def test_encoder_against_reference_golden_outputs(att):
    """The reference's builder-made 2-layer causal-linear encoder (gelu, final norm, randomised
    LayerNorm weights): its state_dict loads into the encoder here by name, and the outputs
    for a full-length and a ragged batch must match.  Heads of 8 dimensions: the odd-shape
    kernels run inside."""
    m = att.masking
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                             "encoder_causal_linear.npz"))
    n_layers, n_heads, qd, vd, ffn = (int(v) for v in z["config"])
    enc = att.build_causal_linear_encoder(n_layers=n_layers, n_heads=n_heads,
                                          query_dimensions=qd, value_dimensions=vd,
                                          feed_forward_dimensions=ffn, activation="gelu",
                                          final_normalization=True)
    state = {k[len("param:"):]: torch.from_numpy(z[k]) for k in z.files if k.startswith("param:")}
    assert set(state) == set(enc.state_dict()), "parameter names differ from the reference's"
    enc.load_state_dict(state, strict=True)
    enc = enc.cuda().eval()
    x = torch.from_numpy(z["x"]).cuda()
    L = x.shape[1]
    mask = m.TriangularCausalMask(L, device="cuda")
    with torch.no_grad():
        y_full = enc(x, attn_mask=mask)
        y_ragged = enc(x, attn_mask=mask,
                       length_mask=m.LengthMask(torch.from_numpy(z["lengths"]).cuda(), max_len=L))
    err_full = (y_full.cpu() - torch.from_numpy(z["y_full"])).abs().max().item()
    err_ragged = (y_ragged.cpu() - torch.from_numpy(z["y_ragged"])).abs().max().item()
    print("encoder vs reference outputs: full %.2e ragged %.2e" % (err_full, err_ragged),
          flush=True)
    assert err_full < 1e-4 and err_ragged < 1e-4


def test_attention_takes_the_reference_constructor_arguments(att):
    """feature_map is a factory called with the query dimensions (feature_maps/base.py:42-53),
    event_dispatcher is accepted (attention/causal_linear_attention.py:47-55)."""
    calls = []

    class Squares(torch.nn.Module):           # an asymmetric map: queries and keys differ
        def __init__(self, query_dims):
            super().__init__()
            calls.append(query_dims)

        def new_feature_map(self, device):
            calls.append(str(device))

        def forward_queries(self, x):
            return x * x + 0.5

        def forward_keys(self, x):
            return x.abs() + 0.25

    m = att.masking
    N, L, H, E, M = 2, 50, 2, 16, 16
    gen = torch.Generator().manual_seed(8)
    q, k, v = (torch.randn(N, L, H, X, generator=gen).cuda() for X in (E, E, M))
    layer = att.CausalLinearAttention(E, feature_map=Squares, eps=1e-5, event_dispatcher="")
    lengths = m.LengthMask(torch.full((N,), L).cuda(), max_len=L)
    out = layer(q, k, v, m.TriangularCausalMask(L, device="cuda"), lengths, lengths)
    assert calls[0] == E and calls[1].startswith("cuda")
    Q, K = (q.double() ** 2 + 0.5), (k.double().abs() + 0.25)
    A = torch.einsum("nlhe,nshe->nhls", Q, K) * torch.tril(
        torch.ones(L, L, dtype=torch.float64, device="cuda"))
    want = torch.einsum("nhls,nshm->nlhm", A / (A.sum(-1, keepdim=True) + 1e-5), v.double())
    assert (out.double() - want).abs().max().item() < 1e-5
