"""Encoder blocks around ``CausalLinearAttention`` (for the 8-layer encoder workload).

Own counterparts of ``fast_transformers/attention/attention_layer.py:44-115`` (Q/K/V/out
projections around an inner attention) and ``fast_transformers/transformers.py:21-145``
(post-norm encoder layer, stack with optional final norm).  Parameter names match the
reference modules so that a reference ``state_dict`` loads unchanged.  Plain ``torch.nn``:
the only custom kernel is inside the inner attention.
"""
import torch
import torch.nn.functional as F
from torch.nn import Dropout, LayerNorm, Linear, Module, ModuleList

from ..masking import FullMask, LengthMask, TriangularCausalMask
from .causal_linear_attention import CausalLinearAttention


class AttentionLayer(Module):
    """Project to multi-head queries/keys/values, run the inner attention, project back
    (``attention_layer.py:44-115``)."""

    def __init__(self, attention, d_model, n_heads, d_keys=None, d_values=None,
                 d_model_keys=None):
        super().__init__()
        d_keys = d_keys or (d_model // n_heads)
        d_values = d_values or (d_model // n_heads)
        d_model_keys = d_model_keys or d_model
        self.inner_attention = attention
        self.query_projection = Linear(d_model, d_keys * n_heads)
        self.key_projection = Linear(d_model_keys, d_keys * n_heads)
        self.value_projection = Linear(d_model_keys, d_values * n_heads)
        self.out_projection = Linear(d_values * n_heads, d_model)
        self.n_heads = n_heads

    def forward(self, queries, keys, values, attn_mask, query_lengths, key_lengths):
        N, L, _ = queries.shape
        S = keys.shape[1]
        H = self.n_heads
        q = self.query_projection(queries).view(N, L, H, -1)
        k = self.key_projection(keys).view(N, S, H, -1)
        v = self.value_projection(values).view(N, S, H, -1)
        new_values = self.inner_attention(q, k, v, attn_mask, query_lengths,
                                          key_lengths).reshape(N, L, -1)
        return self.out_projection(new_values)


class TransformerEncoderLayer(Module):
    """Self attention + feed-forward with skip connections, post-norm
    (``transformers.py:21-89``)."""

    def __init__(self, attention, d_model, d_ff=None, dropout=0.1, activation="relu"):
        super().__init__()
        d_ff = d_ff or 4 * d_model
        self.attention = attention
        self.linear1 = Linear(d_model, d_ff)
        self.linear2 = Linear(d_ff, d_model)
        self.norm1 = LayerNorm(d_model)
        self.norm2 = LayerNorm(d_model)
        self.dropout = Dropout(dropout)
        self.activation = getattr(F, activation)

    def forward(self, x, attn_mask=None, length_mask=None):
        N, L = x.shape[0], x.shape[1]
        attn_mask = attn_mask or FullMask(L, device=x.device)
        length_mask = length_mask or LengthMask(x.new_full((N,), L, dtype=torch.int64))
        x = x + self.dropout(self.attention(x, x, x, attn_mask=attn_mask,
                                            query_lengths=length_mask,
                                            key_lengths=length_mask))
        y = x = self.norm1(x)
        y = self.dropout(self.activation(self.linear1(y)))
        y = self.dropout(self.linear2(y))
        return self.norm2(x + y)


class TransformerEncoder(Module):
    """A stack of encoder layers with an optional final norm (``transformers.py:92-145``)."""

    def __init__(self, layers, norm_layer=None):
        super().__init__()
        self.layers = ModuleList(layers)
        self.norm = norm_layer

    def forward(self, x, attn_mask=None, length_mask=None):
        N, L = x.shape[0], x.shape[1]
        attn_mask = attn_mask or FullMask(L, device=x.device)
        length_mask = length_mask or LengthMask(x.new_full((N,), L, dtype=torch.int64))
        for layer in self.layers:
            x = layer(x, attn_mask=attn_mask, length_mask=length_mask)
        if self.norm is not None:
            x = self.norm(x)
        return x


def build_causal_linear_encoder(n_layers=8, n_heads=8, query_dimensions=64,
                                value_dimensions=64, feed_forward_dimensions=1024,
                                dropout=0.1, activation="relu", final_normalization=True):
    """What ``TransformerEncoderBuilder.from_kwargs(attention_type="causal-linear", ...).get()``
    assembles (``builders/transformer_builders.py:219-251``): d_model = n_heads *
    value_dimensions, one ``AttentionLayer(CausalLinearAttention)`` per layer, final
    LayerNorm.  The caller passes ``attn_mask=TriangularCausalMask(L)``."""
    d_model = n_heads * value_dimensions
    layers = [
        TransformerEncoderLayer(
            AttentionLayer(CausalLinearAttention(query_dimensions), d_model, n_heads,
                           d_keys=query_dimensions, d_values=value_dimensions),
            d_model, feed_forward_dimensions, dropout, activation)
        for _ in range(n_layers)
    ]
    return TransformerEncoder(layers, LayerNorm(d_model) if final_normalization else None)


__all__ = ["AttentionLayer", "TransformerEncoderLayer", "TransformerEncoder",
           "build_causal_linear_encoder", "TriangularCausalMask", "LengthMask", "FullMask"]
