"""Writes the golden vectors in this directory from the reference's own CPU extension.

    make -C oracle ref && python tests/golden/make_golden.py

The extension is compiled by oracle/Makefile from
/root/reference/fast_transformers/causal_product/causal_product_cpu.cpp (the file is
compiled where it lies; nothing of it is stored here).  Each ``causal_*.npz`` holds seeded
inputs Q, K, V, G and the outputs ``product``, ``grad_queries``, ``grad_keys``,
``grad_values`` that ``causal_dot_product`` / ``causal_dot_backward``
(causal_product_cpu.cpp:82-209) produced for them, called the way the reference's tests call
them (tests/causal_product/test_causal_product_cpu.py:42-43,62-63).
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402

# name: (N, H, L, E, M, seed, positive_uniform)
CASES = {
    "causal_tiny_e3_m2": (1, 1, 5, 3, 2, 11, False),
    "causal_e25_m64": (1, 2, 37, 25, 64, 12, True),       # odd E as in the recurrent test
    "causal_e10_m255": (1, 1, 33, 10, 255, 13, True),      # widest odd M the CPU test draws
    "causal_e64_m64_l130": (1, 2, 130, 64, 64, 14, False),  # L just over two 64-chunks
    "causal_e32_m128": (1, 2, 70, 32, 128, 15, False),     # asymmetric heads
    "causal_e200_m17": (1, 1, 20, 200, 17, 16, True),
}


def main():
    ref = oracle.load_reference_extension()
    for name, (N, H, L, E, M, seed, pos) in CASES.items():
        Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed, positive_uniform=pos)
        out = torch.zeros(N, H, L, M)
        ref.causal_dot_product(Q, K, V, out)
        gq, gk, gv = torch.zeros_like(Q), torch.zeros_like(K), torch.zeros_like(V)
        ref.causal_dot_backward(Q, K, V, G, gq, gk, gv)
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            Q=Q.numpy(), K=K.numpy(), V=V.numpy(), G=G.numpy(), product=out.numpy(),
            grad_queries=gq.numpy(), grad_keys=gk.numpy(), grad_values=gv.numpy())
        print(name, os.path.getsize(os.path.join(HERE, name + ".npz")), "bytes")


if __name__ == "__main__":
    main()
