"""TEST INFRASTRUCTURE ONLY: CPU checker for the causal linear-attention product.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped package never does.

Contents
--------
* ``causal_dot_product`` / ``causal_dot_backward``: ctypes bindings to
  ``liboracle_causal.so`` (``causal_product_oracle.c``), the C restatement of
  ``fast_transformers/causal_product/causal_product_cpu.cpp:82-209``.  They keep
  the reference's calling convention: caller-allocated outputs, written in place
  (``causal_product_cpu.cpp:82-87,133-141``).  float32 and float64 tensors.
* ``dense_forward`` / ``dense_backward``: the closed forms ``tril(Q K^T) V`` and
  their gradients, i.e. what the reference's own tests compare against
  (``tests/causal_product/test_causal_product_cpu.py:45-47,65-70``).
* ``forward_with_state``: the forward with the running state handed in and out
  (the ``Si`` of the reference's step-wise module).
* ``recurrent_forward``: the step-wise einsum form of
  ``fast_transformers/recurrent/attention/self_attention/linear_attention.py:79-88``
  without the feature map and normaliser.
* ``causal_linear_attention``: the caller of the op restated, feature map, key-length mask
  and normaliser included (attention/causal_linear_attention.py:71-104).
* ``make_inputs``: the seeded input generator for the measured configurations
  (Q, K = elu(x)+1 with x ~ N(0,1); V, G ~ N(0,1); draw order x_q, x_k, V, G).
* ``load_reference_extension``: the reference's own CPU extension compiled by
  ``make -C oracle ref`` into ``oracle/_ref`` (absent unless built).
"""
import ctypes
import importlib.util
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_causal.so")
_REF_PATH = os.path.join(_HERE, "_ref", "causal_product_cpu_ref.so")
_lib = None


def build(with_reference=None):
    """Compile the C restatement (and the reference extension when its sources exist)."""
    subprocess.check_call(["make", "-C", _HERE, "-s", "-B", "all"])
    if with_reference is None:
        with_reference = os.path.exists(
            "/root/reference/fast_transformers/causal_product/causal_product_cpu.cpp")
    if with_reference:
        subprocess.check_call(["make", "-C", _HERE, "-s", "ref"])


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build(with_reference=False)
        _lib = ctypes.CDLL(_LIB_PATH)
        i64p = ctypes.POINTER(ctypes.c_int64)
        for sfx in ("f32", "f64"):
            f = getattr(_lib, "oracle_causal_dot_product_" + sfx)
            f.restype = ctypes.c_int
            f.argtypes = [ctypes.c_void_p, i64p] * 4 + [ctypes.c_int] * 5
            st = getattr(_lib, "oracle_causal_dot_product_state_" + sfx)
            st.restype = ctypes.c_int
            st.argtypes = ([ctypes.c_void_p, i64p] * 3 + [ctypes.c_void_p] +
                           [ctypes.c_void_p, i64p] + [ctypes.c_void_p] + [ctypes.c_int] * 5)
            b = getattr(_lib, "oracle_causal_dot_backward_" + sfx)
            b.restype = ctypes.c_int
            b.argtypes = [ctypes.c_void_p, i64p] * 7 + [ctypes.c_int] * 5
    return _lib


def _arg(t):
    strides = (ctypes.c_int64 * 4)(*t.stride())
    return ctypes.c_void_p(t.data_ptr()), strides


def _suffix(*tensors):
    dt = tensors[0].dtype
    for t in tensors:
        if t.dtype != dt or t.device.type != "cpu" or t.dim() != 4:
            raise RuntimeError("oracle: expected 4-d CPU tensors of one dtype")
    if dt == torch.float32:
        return "f32"
    if dt == torch.float64:
        return "f64"
    raise RuntimeError("oracle: float32 or float64 only")


def causal_dot_product(queries, keys, values, product):
    """In-place forward with the reference's native signature (cpp:82-87)."""
    lib = _load()
    sfx = _suffix(queries, keys, values, product)
    N, H, L, E = queries.shape
    M = values.shape[3]
    assert keys.shape == (N, H, L, E) and values.shape == (N, H, L, M)
    assert product.shape == (N, H, L, M)
    args = []
    for t in (queries, keys, values, product):
        args.extend(_arg(t))
    rc = getattr(lib, "oracle_causal_dot_product_" + sfx)(*args, N, H, L, E, M)
    if rc != 0:
        raise RuntimeError("oracle forward failed (%d)" % rc)


def causal_dot_backward(queries, keys, values, grad_out, grad_queries, grad_keys, grad_values):
    """In-place backward with the reference's native signature (cpp:133-141)."""
    lib = _load()
    sfx = _suffix(queries, keys, values, grad_out, grad_queries, grad_keys, grad_values)
    N, H, L, E = queries.shape
    M = values.shape[3]
    assert grad_out.shape == (N, H, L, M)
    assert grad_queries.shape == (N, H, L, E) and grad_keys.shape == (N, H, L, E)
    assert grad_values.shape == (N, H, L, M)
    args = []
    for t in (queries, keys, values, grad_out, grad_queries, grad_keys, grad_values):
        args.extend(_arg(t))
    rc = getattr(lib, "oracle_causal_dot_backward_" + sfx)(*args, N, H, L, E, M)
    if rc != 0:
        raise RuntimeError("oracle backward failed (%d)" % rc)


def forward_with_state(Q, K, V, initial_state=None):
    """(product, final_state) with the running state handed in and out; the state is the
    ``Si`` of recurrent/attention/self_attention/linear_attention.py:63-66,79-80."""
    lib = _load()
    sfx = _suffix(Q, K, V)
    N, H, L, E = Q.shape
    M = V.shape[3]
    out = torch.empty(N, H, L, M, dtype=Q.dtype)
    s1 = torch.empty(N, H, E, M, dtype=Q.dtype)
    s0p = None
    if initial_state is not None:
        s0 = initial_state.to(Q.dtype).contiguous()
        assert s0.shape == (N, H, E, M)
        s0p = ctypes.c_void_p(s0.data_ptr())
    args = []
    for t in (Q, K, V):
        args.extend(_arg(t))
    rc = getattr(lib, "oracle_causal_dot_product_state_" + sfx)(
        *args, s0p, *_arg(out), ctypes.c_void_p(s1.data_ptr()), N, H, L, E, M)
    if rc != 0:
        raise RuntimeError("oracle stateful forward failed (%d)" % rc)
    return out, s1


def forward(Q, K, V):
    """Allocate-and-return convenience around ``causal_dot_product``."""
    out = torch.empty(Q.shape[:3] + (V.shape[3],), dtype=Q.dtype)
    causal_dot_product(Q, K, V, out)
    return out


def backward(Q, K, V, G):
    dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    causal_dot_backward(Q, K, V, G, dQ, dK, dV)
    return dQ, dK, dV


def dense_forward(Q, K, V):
    """out = tril(Q K^T) V   (tests/causal_product/test_causal_product_cpu.py:45-47)."""
    L = Q.shape[2]
    A = torch.einsum("nhle,nhse->nhls", Q, K)
    A = A * torch.tril(torch.ones(L, L, dtype=Q.dtype, device=Q.device))
    return torch.einsum("nhls,nhsm->nhlm", A, V)


def dense_backward(Q, K, V, G):
    """dQ = tril(G V^T) K ; dK = tril(G V^T)^T Q ; dV = tril(Q K^T)^T G."""
    L = Q.shape[2]
    mask = torch.tril(torch.ones(L, L, dtype=Q.dtype, device=Q.device))
    B = torch.einsum("nhlm,nhsm->nhls", G, V) * mask
    A = torch.einsum("nhle,nhse->nhls", Q, K) * mask
    dQ = torch.einsum("nhls,nhse->nhle", B, K)
    dK = torch.einsum("nhls,nhle->nhse", B, Q)
    dV = torch.einsum("nhls,nhlm->nhsm", A, G)
    return dQ, dK, dV


def recurrent_forward(Q, K, V):
    """Step-wise state form (recurrent/attention/self_attention/linear_attention.py:79-88)."""
    N, H, L, E = Q.shape
    M = V.shape[3]
    S = torch.zeros(N, H, E, M, dtype=Q.dtype)
    out = torch.empty(N, H, L, M, dtype=Q.dtype)
    for l in range(L):
        S = S + torch.einsum("nhe,nhm->nhem", K[:, :, l], V[:, :, l])
        out[:, :, l] = torch.einsum("nhe,nhem->nhm", Q[:, :, l], S)
    return out


def causal_linear_attention(queries, keys, values, key_lengths=None, eps=1e-6):
    """``CausalLinearAttention.forward`` with the default feature map, restated
    (attention/causal_linear_attention.py:71-104; feature_maps/base.py:71-73) over
    ``(N, L, H, E)`` / ``(N, L, H, M)`` CPU tensors, equal numbers of queries and keys;
    ``key_lengths``: N integers, or None when every key counts.

    phi = elu + 1 on queries and keys (:75-76); keys at or beyond the length are zeroed
    (:83); Z = 1 / (q . cumsum(k) + eps) (:95); the unnormalised rows come from the C
    restatement of the native op on (N, H, L, X) copies (:19-24, :98-102); result rows are
    scaled by Z (:104).

    Pinned by: the outputs of the reference module itself stored in
    tests/golden/attention_causal_linear.npz; the dense normalised closed form of the
    reference's API test (tests/causal_product/test_causal_product.py:34-52) and the
    step-wise form (recurrent/attention/self_attention/linear_attention.py:55-88), both in
    tests/test_oracle.py."""
    Q = torch.nn.functional.elu(queries) + 1
    K = torch.nn.functional.elu(keys) + 1
    N, L = Q.shape[0], Q.shape[1]
    if key_lengths is not None:
        keep = torch.arange(L)[None, :] < torch.as_tensor(key_lengths).reshape(N, 1)
        K = K * keep.to(K.dtype)[:, :, None, None]
    Z = 1 / (torch.einsum("nlhi,nlhi->nlh", Q, K.cumsum(1)) + eps)
    product = forward(Q.permute(0, 2, 1, 3).contiguous(), K.permute(0, 2, 1, 3).contiguous(),
                      values.permute(0, 2, 1, 3).contiguous())
    return product.permute(0, 2, 1, 3).contiguous() * Z[:, :, :, None]


def make_inputs(N, H, L, E, M, seed, dtype=torch.float32, positive_uniform=False):
    """Seeded inputs.  Default: Q, K = elu(x)+1, x ~ N(0,1); V, G ~ N(0,1).
    ``positive_uniform`` gives the reference tests' distribution, all U[0,1)
    (tests/causal_product/test_causal_product_cpu.py:39-41,57-60)."""
    gen = torch.Generator().manual_seed(seed)
    if positive_uniform:
        Q = torch.rand(N, H, L, E, generator=gen)
        K = torch.rand(N, H, L, E, generator=gen)
        V = torch.rand(N, H, L, M, generator=gen)
        G = torch.rand(N, H, L, M, generator=gen)
    else:
        Q = torch.nn.functional.elu(torch.randn(N, H, L, E, generator=gen)) + 1
        K = torch.nn.functional.elu(torch.randn(N, H, L, E, generator=gen)) + 1
        V = torch.randn(N, H, L, M, generator=gen)
        G = torch.randn(N, H, L, M, generator=gen)
    return tuple(t.to(dtype) for t in (Q, K, V, G))


def reference_extension_available():
    return os.path.exists(_REF_PATH)


def load_reference_extension():
    """The reference's CPU extension built by ``make -C oracle ref`` (module with
    ``causal_dot_product`` and ``causal_dot_backward``,
    causal_product_cpu.cpp:212-225)."""
    if not os.path.exists(_REF_PATH):
        raise RuntimeError("oracle/_ref is not built (run `make -C oracle ref` where the "
                           "reference sources are present)")
    spec = importlib.util.spec_from_file_location("causal_product_cpu_ref", _REF_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod
