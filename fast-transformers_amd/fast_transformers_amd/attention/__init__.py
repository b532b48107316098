"""Causal linear attention module and the encoder blocks around it (the caller side of the
hot path)."""
from .causal_linear_attention import CausalLinearAttention, causal_linear, elu_feature_map
from .encoder import AttentionLayer, TransformerEncoderLayer, TransformerEncoder, \
    build_causal_linear_encoder
