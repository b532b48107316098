"""Writes tests/golden/encoder_causal_linear.npz and tests/golden/attention_causal_linear.npz
from the reference's own modules.

    python tests/golden/make_encoder_golden.py          (build container only)

What it pins: the block structure of a builder-made causal-linear encoder -- projection
order and head split (attention/attention_layer.py:61-115), feature map, key-length masking
and normaliser (attention/causal_linear_attention.py:71-104), residual / post-norm order and
feed-forward (transformers.py:55-89), final norm (transformers.py:115-145), module and
parameter names (builders/transformer_builders.py:219-251) -- none of which a closed form
or a test of the reference fixes.

How: the reference package imports all of its seven CPU extensions
(attention/__init__.py:10-21, setup.py:84-134), and /root/reference is read-only.  The
script therefore compiles the seven ``*_cpu.cpp`` files with g++ from where they lie into a
scratch package under /tmp whose ``.py`` files are symbolic links into /root/reference,
imports ``fast_transformers.builders`` from there, builds a 2-layer encoder
(d_model 32, 4 heads, feed-forward 64) with ``TransformerEncoderBuilder``, and stores its
``state_dict``, two inputs (full length, and ragged lengths) and the outputs of
``encoder(x, attn_mask=TriangularCausalMask(L), length_mask=...)``.  Nothing of the
reference is stored in this repository; the fixture is data (< 100 KB).

The second file pins the attention module alone (attention/causal_linear_attention.py:71-104
with the default feature map): raw queries and keys with both signs (so that both branches
of elu(x) + 1 are taken), values, ragged key lengths, and the module's output, at two shapes
(E = M = 8 over 37 positions; E = 64, M = 32 over 40 positions).
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = "/root/reference"
SCRATCH = "/tmp/ft_reference_pkg"

EXTENSIONS = [
    "hashing/hash_cpu",
    "aggregate/aggregate_cpu",
    "clustering/hamming/cluster_cpu",
    "sparse_product/sparse_product_cpu",
    "sparse_product/clustered_sparse_product_cpu",
    "causal_product/causal_product_cpu",
    "local_product/local_product_cpu",
]


def shadow_package():
    """A package directory under /tmp: links to the reference's .py files plus the built
    extension modules next to them."""
    src_root = os.path.join(REFERENCE, "fast_transformers")
    dst_root = os.path.join(SCRATCH, "fast_transformers")
    for dirpath, _, files in os.walk(src_root):
        rel = os.path.relpath(dirpath, src_root)
        os.makedirs(os.path.join(dst_root, rel), exist_ok=True)
        for f in files:
            if f.endswith(".py"):
                dst = os.path.join(dst_root, rel, f)
                if not os.path.lexists(dst):
                    os.symlink(os.path.join(dirpath, f), dst)
    return dst_root


def build_extension(dst_root, ext):
    name = os.path.basename(ext)
    out = os.path.join(dst_root, ext + ".so")
    if os.path.exists(out):
        return out
    torch_dir = os.path.dirname(torch.__file__)
    cmd = ["g++", "-O2", "-DNDEBUG", "-fopenmp", "-ffast-math", "-fPIC", "-shared", "-std=c++17",
           "-DTORCH_EXTENSION_NAME=" + name, "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(torch_dir, "include"),
           "-I" + os.path.join(torch_dir, "include/torch/csrc/api/include"),
           "-I" + sysconfig.get_paths()["include"],
           os.path.join(REFERENCE, "fast_transformers", ext + ".cpp"), "-o", out,
           "-L" + os.path.join(torch_dir, "lib"), "-Wl,-rpath," + os.path.join(torch_dir, "lib"),
           "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python"]
    subprocess.check_call(cmd)
    return out


def main():
    dst_root = shadow_package()
    with ThreadPoolExecutor(4) as pool:
        list(pool.map(lambda e: build_extension(dst_root, e), EXTENSIONS))
    sys.path.insert(0, SCRATCH)
    from fast_transformers.builders import TransformerEncoderBuilder
    from fast_transformers.masking import LengthMask, TriangularCausalMask

    torch.manual_seed(2024)
    n_layers, n_heads, qd, vd, ffn = 2, 4, 8, 8, 64
    encoder = TransformerEncoderBuilder.from_kwargs(
        n_layers=n_layers, n_heads=n_heads, query_dimensions=qd, value_dimensions=vd,
        feed_forward_dimensions=ffn, attention_type="causal-linear", activation="gelu",
        dropout=0.1, final_normalization=True).get().eval()
    # make the norms non-trivial, so that a wrong norm order cannot hide behind weight 1, bias 0
    with torch.no_grad():
        for name, p in encoder.named_parameters():
            if "norm" in name:
                p.add_(0.3 * torch.randn_like(p))
    N, L, D = 2, 28, n_heads * vd
    x = torch.rand(N, L, D)
    lengths = torch.tensor([L, 19])
    with torch.no_grad():
        y_full = encoder(x, attn_mask=TriangularCausalMask(L))
        y_ragged = encoder(x, attn_mask=TriangularCausalMask(L),
                           length_mask=LengthMask(lengths, max_len=L))
    arrays = {"param:" + k: v.numpy() for k, v in encoder.state_dict().items()}
    arrays.update(x=x.numpy(), lengths=lengths.numpy(), y_full=y_full.numpy(),
                  y_ragged=y_ragged.numpy(),
                  config=np.array([n_layers, n_heads, qd, vd, ffn]))
    out = os.path.join(HERE, "encoder_causal_linear.npz")
    np.savez_compressed(out, **arrays)
    print(out, os.path.getsize(out), "bytes;", len(arrays), "arrays")
    for k in sorted(arrays):
        print("  ", k, arrays[k].shape)

    from fast_transformers.attention import CausalLinearAttention
    arrays = {}
    for tag, (N, L, H, E, M, lens) in {"a": (2, 37, 3, 8, 8, [37, 20]),
                                        "b": (2, 40, 1, 64, 32, [40, 13])}.items():
        att = CausalLinearAttention(E).eval()
        q = 1.5 * torch.randn(N, L, H, E)
        k = 1.5 * torch.randn(N, L, H, E)
        v = torch.randn(N, L, H, M)
        lengths = torch.tensor(lens)
        with torch.no_grad():
            y = att(q, k, v, TriangularCausalMask(L), LengthMask(torch.full((N,), L), max_len=L),
                    LengthMask(lengths, max_len=L))
        arrays.update({tag + "_q": q.numpy(), tag + "_k": k.numpy(), tag + "_v": v.numpy(),
                       tag + "_lengths": lengths.numpy(), tag + "_y": y.numpy(),
                       tag + "_eps": np.array(att.eps)})
    out = os.path.join(HERE, "attention_causal_linear.npz")
    np.savez_compressed(out, **arrays)
    print(out, os.path.getsize(out), "bytes;", len(arrays), "arrays")


if __name__ == "__main__":
    main()
