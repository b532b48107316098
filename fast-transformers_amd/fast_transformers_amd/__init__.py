"""MI355X-native causal linear-attention product.

Drop-in for ``fast_transformers.causal_product`` (reference
``fast_transformers/causal_product/__init__.py:20-78``): the same
``causal_dot_product(Q, K, V)`` autograd function over ``(N, H, L, E)`` /
``(N, H, L, M)`` tensors, computed by hand-written gfx950 kernels behind the C ABI
declared in ``include/ftc_causal_product.h``.
"""
__version__ = "0.1.0"
