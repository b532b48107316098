"""Causally masked linear attention on top of the MI355X ``causal_dot_product``.

Own counterpart of ``fast_transformers/attention/causal_linear_attention.py:19-104``: same
constructor arguments, same ``forward(queries, keys, values, attn_mask, query_lengths,
key_lengths)`` over ``(N, L, H, E)`` tensors, same equations (feature map ``elu(x)+1``
``feature_maps/base.py:71-73``; key-length masking ``:83``; normaliser
``Z = 1 / (q . cumsum(k) + eps)`` ``:95``; result ``V' * Z`` ``:104``).

One difference in mechanics: the reference makes four ``permute().contiguous()`` copies
around the native call (``:19-24``).  The kernels here take any N/H/L strides, so the
``(N, L, H, X)`` tensors are handed over as permuted views and the product is written
straight into ``(N, L, H, M)`` storage.
"""
import torch
from torch.nn import Module

from ..causal_product import causal_dot_product_hip, causal_dot_backward_hip


def elu_feature_map(x):
    """phi(x) = elu(x) + 1 (``feature_maps/base.py:71-73``)."""
    return torch.nn.functional.elu(x) + 1


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
        gQ, gK, gV = (torch.empty(t.shape, device=t.device, dtype=t.dtype) for t in (Q, K, V))
        G = grad_out if grad_out.dtype == torch.float32 else grad_out.float()
        causal_dot_backward_hip(Q.permute(0, 2, 1, 3), K.permute(0, 2, 1, 3),
                                V.permute(0, 2, 1, 3), G.contiguous().permute(0, 2, 1, 3),
                                gQ.permute(0, 2, 1, 3), gK.permute(0, 2, 1, 3),
                                gV.permute(0, 2, 1, 3))
        return gQ, gK, gV


def causal_linear(Q, K, V):
    """(N, L, H, E), (N, L, H, E), (N, L, H, M) -> (N, L, H, M); reference ``:19-24``."""
    return _CausalLinearNLH.apply(Q, K, V)


class CausalLinearAttention(Module):
    """Causally masked attention with feature maps in O(L D^2) (reference ``:27-104``).

    Arguments: ``query_dimensions`` (kept for signature compatibility), ``feature_map`` (a
    callable applied to queries and keys, default ``elu(x)+1``), ``eps`` (default 1e-6).
    """

    def __init__(self, query_dimensions, feature_map=None, eps=1e-6):
        super().__init__()
        self.query_dimensions = query_dimensions
        self.feature_map = feature_map or elu_feature_map
        self.eps = eps

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

    def forward(self, queries, keys, values, attn_mask, query_lengths, key_lengths):
        Q = self.feature_map(queries)
        K = self.feature_map(keys)
        if not attn_mask.lower_triangular:
            raise RuntimeError("CausalLinearAttention only supports full lower triangular masks")
        K = K * key_lengths.float_matrix[:, :, None, None]
        K, values = self._make_sizes_compatible(Q, K, values)
        Z = 1 / (torch.einsum("nlhi,nlhi->nlh", Q, K.cumsum(1)) + self.eps)
        V = causal_linear(Q, K, values)
        return V * Z[:, :, :, None]
