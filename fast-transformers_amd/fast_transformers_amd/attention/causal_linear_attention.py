"""Causally masked linear attention on top of the MI355X ``causal_dot_product``.

Own counterpart of ``fast_transformers/attention/causal_linear_attention.py:19-104``: same
constructor arguments (feature-map factory, ``eps``, ``event_dispatcher``), same ``forward(queries, keys, values, attn_mask, query_lengths,
key_lengths)`` over ``(N, L, H, E)`` tensors, same equations (feature map ``elu(x)+1``
``feature_maps/base.py:71-73``; key-length masking ``:83``; normaliser
``Z = 1 / (q . cumsum(k) + eps)`` ``:95``; result ``V' * Z`` ``:104``).

Two differences in mechanics.  The reference makes four ``permute().contiguous()`` copies
around the native call (``:19-24``); the kernels here take any N/H/L strides, so the
``(N, L, H, X)`` tensors are handed over as permuted views and the product is written
straight into ``(N, L, H, M)`` storage.  And the normaliser's ``q_l . sum_{j<=l} k_j`` is
the same causal product with a column of ones for values, so it is a second call of the
operator instead of a cumulative sum over L followed by a batched dot product (which on
this stack cost ten and fifty times the operator itself).

When nothing has to be differentiated (eval, ``torch.no_grad``) and the feature map is the
default one, the whole body of ``forward`` -- both feature maps, the key-length mask, the
product, the normaliser and the final scale -- is one launch of
``ftc_causal_linear_attention`` (head dimensions 32 or 64, float32), and training on
``CausalLinearAttentionFunction``, whose backward is one launch sequence of its own
(``ftc_causal_linear_attention_backward``).  Other sizes and feature maps keep the composition
above, whose pieces autograd differentiates.
"""
import torch
from torch.nn import Module

from ..causal_product import causal_dot_product_hip, causal_dot_backward_hip, \
    causal_linear_attention_hip, fused_attention_covers, CausalLinearAttentionFunction


class ActivationFunctionFeatureMap(Module):
    """An element-wise feature map behind the reference's feature-map protocol
    (``feature_maps/base.py:19-73``): attention modules receive a *factory* that is called
    with the query dimensions and returns an object with ``new_feature_map(device)``,
    ``forward_queries(x)`` and ``forward_keys(x)``."""

    def __init__(self, query_dims, activation_function):
        super().__init__()
        self.query_dims = query_dims
        self.activation_function = activation_function

    def new_feature_map(self, device):
        return

    def forward_queries(self, x):
        return self(x)

    def forward_keys(self, x):
        return self(x)

    def forward(self, x):
        return self.activation_function(x)

    @classmethod
    def factory(cls, *args, **kwargs):
        def inner(query_dims):
            return cls(query_dims, *args, **kwargs)
        return inner


def _elu_plus_one(x):
    return torch.nn.functional.elu(x) + 1


# phi(x) = elu(x) + 1 as a feature-map factory (``feature_maps/base.py:71-73``)
elu_feature_map = ActivationFunctionFeatureMap.factory(_elu_plus_one)


class _CausalLinearNLH(torch.autograd.Function):
    """``causal_dot_product`` over (N, L, H, X) tensors without layout copies."""

    @staticmethod
    def forward(ctx, Q, K, V):
        ctx.save_for_backward(Q, K, V)
        N, L, H, _ = Q.shape
        out = torch.empty((N, L, H, V.shape[3]), device=Q.device, dtype=torch.float32)
        causal_dot_product_hip(Q.detach().permute(0, 2, 1, 3), K.detach().permute(0, 2, 1, 3),
                               V.detach().permute(0, 2, 1, 3), out.permute(0, 2, 1, 3))
        return out

    @staticmethod
    def backward(ctx, grad_out):
        Q, K, V = ctx.saved_tensors
        # gradients nobody asked for (the normaliser's column of ones) are not computed
        gQ, gK, gV = (torch.empty(t.shape, device=t.device, dtype=t.dtype) if need else None
                      for t, need in zip((Q, K, V), ctx.needs_input_grad))
        G = grad_out if grad_out.dtype == torch.float32 else grad_out.float()
        causal_dot_backward_hip(Q.permute(0, 2, 1, 3), K.permute(0, 2, 1, 3),
                                V.permute(0, 2, 1, 3), G.contiguous().permute(0, 2, 1, 3),
                                *(t.permute(0, 2, 1, 3) if t is not None else None
                                  for t in (gQ, gK, gV)))
        return gQ, gK, gV


_ONES_WIDTH = 32  # the narrowest value width the matrix-core kernels take
_ones_rows = {}


def _ones_column(N, L, H, device):
    """An (N, L, H, 32) view whose column 0 is one and whose other columns are zero, backed
    by a single (L, 32) buffer (zero strides over N and H)."""
    key = (device, L)
    rows = _ones_rows.get(key)
    if rows is None:
        rows = torch.zeros(L, _ONES_WIDTH, device=device, dtype=torch.float32)
        rows[:, 0] = 1
        _ones_rows[key] = rows
    return rows[None, :, None, :].expand(N, L, H, _ONES_WIDTH)


def causal_linear(Q, K, V):
    """(N, L, H, E), (N, L, H, E), (N, L, H, M) -> (N, L, H, M); reference ``:19-24``."""
    return _CausalLinearNLH.apply(Q, K, V)


class CausalLinearAttention(Module):
    """Causally masked attention with feature maps in O(L D^2) (reference ``:27-104``).

    Arguments as in the reference (``:47-55``): ``query_dimensions``; ``feature_map``, a
    factory called with the query dimensions that returns a feature map object (default
    ``elu_feature_map``; any factory of the reference's ``feature_maps`` package fits);
    ``eps`` (default 1e-6); ``event_dispatcher``, accepted and kept for signature
    compatibility (the reference stores a dispatcher here and never dispatches through it,
    ``:55``).
    """

    def __init__(self, query_dimensions, feature_map=None, eps=1e-6, event_dispatcher=""):
        super().__init__()
        self.feature_map = (feature_map(query_dimensions) if feature_map
                            else elu_feature_map(query_dimensions))
        self.eps = eps
        self.event_dispatcher = event_dispatcher

    @staticmethod
    def _make_sizes_compatible(Q, K, V):
        """Slice or zero-pad the keys to the number of queries (reference ``:57-69``).  The
        values follow the keys: positions beyond the queries are never read, and padded
        keys are zero, so padded values contribute nothing."""
        L, S = Q.shape[1], K.shape[1]
        if L == S:
            return K, V
        if L < S:
            return K[:, :L], V[:, :L]
        N, _, H, E = K.shape
        M = V.shape[3]
        return (torch.cat([K, K.new_zeros(N, L - S, H, E)], dim=1),
                torch.cat([V, V.new_zeros(N, L - S, H, M)], dim=1))

    def _fused_forward(self, queries, keys, values, key_lengths):
        """The whole forward in one launch (feature map, key-length mask, product,
        normaliser) when a fused kernel covers the sizes -- with its own backward (one
        element-wise pass, the three gradient scans, one prefix-sum pass) when something has
        to be differentiated; None otherwise."""
        fm = self.feature_map
        if not (isinstance(fm, ActivationFunctionFeatureMap)
                and fm.activation_function is _elu_plus_one):
            return None
        if queries.shape[1] != keys.shape[1] or keys.shape[1] != values.shape[1]:
            return None
        qv, kv, vv = (t.permute(0, 2, 1, 3) for t in (queries, keys, values))
        if not fused_attention_covers(qv, vv, kv):
            return None
        lengths = getattr(key_lengths, "lengths", None)
        if lengths is None:  # not a length mask: the composition multiplies by its matrix
            return None
        lengths = lengths.to(device=queries.device, dtype=torch.int64).contiguous()
        if torch.is_grad_enabled() and (queries.requires_grad or keys.requires_grad
                                        or values.requires_grad):
            return CausalLinearAttentionFunction.apply(qv, kv, vv, lengths, self.eps).permute(0, 2, 1, 3)
        N, L, H, _ = queries.shape
        out = torch.empty((N, L, H, values.shape[3]), device=queries.device, dtype=torch.float32)
        causal_linear_attention_hip(qv, kv, vv, lengths, self.eps, out.permute(0, 2, 1, 3))
        return out

    def forward(self, queries, keys, values, attn_mask, query_lengths, key_lengths):
        if not attn_mask.lower_triangular:
            raise RuntimeError("CausalLinearAttention only supports full lower triangular masks")
        fused = self._fused_forward(queries, keys, values, key_lengths)
        if fused is not None:
            return fused
        self.feature_map.new_feature_map(queries.device)
        Q = self.feature_map.forward_queries(queries)
        K = self.feature_map.forward_keys(keys)
        K = K * key_lengths.float_matrix[:, :, None, None]
        K, values = self._make_sizes_compatible(Q, K, values)
        # q_l . cumsum(k)_l  ==  sum_{j<=l} (q_l . k_j) * 1
        N, L, H, _ = Q.shape
        denominator = causal_linear(Q, K, _ones_column(N, L, H, Q.device))[..., 0]
        Z = 1 / (denominator + self.eps)
        V = causal_linear(Q, K, values)
        return V * Z[:, :, :, None]
