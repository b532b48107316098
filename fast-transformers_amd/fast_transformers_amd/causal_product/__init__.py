"""``causal_dot_product`` on MI355X: same surface as the reference module
``fast_transformers/causal_product/__init__.py``.

* ``CausalDotProduct`` is a ``torch.autograd.Function`` with the class-level
  dispatch tables ``dot`` / ``dot_backward`` keyed by ``device.type``
  (reference ``__init__.py:23-30``).  ROCm PyTorch reports ``"cuda"`` for an AMD
  GPU, so the HIP kernels register under that key.  The ``"cpu"`` entry is a small
  chunked implementation of its own for CPU tensors (plain torch matmuls); the GPU entry
  never falls back to it: without the HIP library a GPU tensor raises.
* The native functions keep the reference's in-place calling convention
  (``causal_product_cpu.cpp:82-87,133-141``): ``causal_dot_product(Q, K, V,
  product)`` and ``causal_dot_backward(Q, K, V, grad_out, grad_Q, grad_K,
  grad_V)`` write caller-allocated tensors and return ``None``.
* Q, K, V are float32 (as in the reference) or bfloat16 (fp32 accumulation).  The
  product is float32 in both cases (``__init__.py:41`` allocates with the default
  dtype) and the gradients have the dtype of their inputs (``__init__.py:59-61``).
"""
import os
import time

import torch

from .. import _native


def _prepare(t, name):
    """The kernels take any N/H/L strides but need unit stride in the last dimension."""
    if t.dim() != 4:
        raise RuntimeError("causal_dot_product: %s must be 4-dimensional (N, H, L, X), got %d-d"
                           % (name, t.dim()))
    if t.device.type != "cuda":
        raise RuntimeError("causal_dot_product: %s is on %s, expected a GPU tensor"
                           % (name, t.device))
    if t.shape[3] > 1 and t.stride(3) != 1:
        return t.contiguous()
    # rows that overlap (an expanded L dimension) would take the slow general path; zero
    # strides over N or H (one sequence shared by chains) are read as they are
    if t.shape[2] > 1 and t.stride(2) < t.shape[3]:
        return t.contiguous()
    return t


def _check_out(t, name):
    if t.dim() != 4 or t.device.type != "cuda":
        raise RuntimeError("causal_dot_product: %s must be a 4-dimensional GPU tensor" % name)
    if t.shape[3] > 1 and t.stride(3) != 1:
        raise RuntimeError("causal_dot_product: output %s must be contiguous in its last "
                           "dimension" % name)
    return t


# One scratch buffer per (device, stream), grown on demand.  The library wants the control
# block at its start zeroed before the first use and restores it after every call, so the
# buffer is allocated zero-filled once and then handed to every later call on that stream.
#
# The error word of a workspace (byte 8 of the control block) is non-zero after a call that
# was cut short.  Reading it means waiting for the GPU, so the wrapper does that only where it
# is asked for (``check_workspaces()``; after every call when FTC_CHECK=1 is set in the
# environment) or cheap (before a cached workspace is replaced by a larger one).  Between
# those it watches without waiting: at most every ``_PROBE_INTERVAL_S`` seconds a call leaves
# an asynchronous copy of the error word to pinned host memory behind it on its stream, and a
# later call that finds the copy finished (an event query) reads the word and raises.
_workspaces = {}
_ws_bytes = {}            # (query, N, H, L, E, M, dtype code) -> bytes: sizes repeat call after call
_probes = {}              # workspace key -> [pinned word, event or None, time of the last probe]
_PROBE_INTERVAL_S = 0.01


class _NoGuard:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _device_guard(device):
    """Make `device` current for the call -- at no cost when it already is."""
    index = device.index
    if index is None or index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(index)


def _workspace_bytes(query, N, H, L, E, M, code):
    key = (query, N, H, L, E, M, code)
    nbytes = _ws_bytes.get(key)
    if nbytes is None:
        nbytes = _native.check(getattr(_native.load(), query)(N, H, L, E, M, code), query)
        _ws_bytes[key] = nbytes
    return nbytes


def reload_tuning():
    """Make the library read its FTC_* environment variables again (they are read once, at first
    use) and forget the workspace sizes asked for under the old values.  A debugging aid: call
    it with no work in flight."""
    _native.check(_native.load().ftc_tuning_reload(), "ftc_tuning_reload")
    _ws_bytes.clear()


def _workspace(nbytes, device, stream=None):
    if nbytes <= 0:
        return None, 0
    if stream is None:
        stream = torch.cuda.current_stream(device).cuda_stream
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            check_workspaces()  # the old buffer's last word on the calls made with it
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
        _probes.pop(key, None)
    _watch(key, ws)
    return ws, ws.numel()


def _watch(key, ws):
    """Look at a finished probe of this workspace, if there is one; otherwise nothing."""
    probe = _probes.get(key)
    if probe is None or probe[1] is None:
        return
    if not torch.cuda.is_current_stream_capturing() and probe[1].query():
        probe[1] = None
        if int(probe[0].item()) != 0:
            check_workspaces()   # synchronises, resets the control block and raises


def _after_call(ws=None, stream=None):
    if os.environ.get("FTC_CHECK", "0") not in ("", "0"):
        # the check synchronises, which a capturing stream does not allow: a captured call is
        # checked by the first eager call after the replays, or by check_workspaces()
        if not torch.cuda.is_current_stream_capturing():
            check_workspaces()
        return
    if ws is None:
        return
    # leave a probe behind this call when the last one is old enough and has been read
    now = time.monotonic()
    if stream is None:
        stream = torch.cuda.current_stream(ws.device).cuda_stream
    key = (ws.device.index, stream)
    probe = _probes.get(key)
    if probe is not None and (probe[1] is not None or now - probe[2] < _PROBE_INTERVAL_S):
        return
    if torch.cuda.is_current_stream_capturing():
        return
    if probe is None:
        probe = _probes[key] = [torch.zeros(1, dtype=torch.int32).pin_memory(), None, 0.0]
    probe[0].copy_(ws[8:12].view(torch.int32), non_blocking=True)
    ev = torch.cuda.Event()
    ev.record()
    probe[1], probe[2] = ev, now


def workspace_error_words():
    """Error word of every cached workspace (synchronises).  All zero unless a wavefront
    gave up waiting for another one, which a correct launch never does."""
    return {key: int(ws[8:12].view(torch.int32).item()) for key, ws in _workspaces.items()}


def check_workspaces():
    """Synchronise and raise if any cached workspace reports that a call was cut short.  The
    control block of such a workspace is cleared first (``ftc_workspace_reset``, on the current
    stream of its device once that device is idle: the stream the workspace was cached for may
    be gone by now), so calls made after the exception start from a clean workspace again: a
    control block left non-zero would make every later call on it stop early with its outputs
    unwritten."""
    bad = {key: word for key, word in workspace_error_words().items() if word != 0}
    if not bad:
        return
    lib = _native.load()
    for (device_index, stream) in bad:
        ws = _workspaces[(device_index, stream)]
        with torch.cuda.device(device_index):
            torch.cuda.synchronize()
            _native.check(lib.ftc_workspace_reset(ws.data_ptr(), ws.numel(),
                                                  torch.cuda.current_stream().cuda_stream),
                          "ftc_workspace_reset")
            torch.cuda.synchronize()
        _probes.pop((device_index, stream), None)
    raise RuntimeError("causal_dot_product: a call was cut short on workspace(s) %s "
                       "(error words %s); its outputs are not valid.  The workspaces have "
                       "been reset." % (sorted(bad), [bad[k] for k in sorted(bad)]))


def causal_dot_product_hip(queries, keys, values, product):
    """In-place forward; replaces the reference's native ``causal_dot_product``
    (``causal_product_cuda.cu:1273-1285``).  Enqueued on the current stream."""
    lib = _native.load()
    q, k, v = (_prepare(t, n) for t, n in
               ((queries, "queries"), (keys, "keys"), (values, "values")))
    out = _check_out(product, "product")
    N, H, L, E = q.shape
    M = v.shape[3]
    with _device_guard(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = _workspace_bytes("ftc_causal_dot_product_workspace_bytes", N, H, L, E, M,
                                  _native.dtype_code(q.dtype))
        ws, nbytes = _workspace(nbytes, q.device, stream)
        dq, dk, dv, do = (_native.describe(t) for t in (q, k, v, out))
        rc = lib.ftc_causal_dot_product(dq, dk, dv, do, ws.data_ptr() if ws is not None else None,
                                        nbytes, stream)
        _native.check(rc, "ftc_causal_dot_product")
        _after_call(ws, stream)


def causal_dot_product_with_state(queries, keys, values, initial_state=None,
                                  return_state=True):
    """The product of a piece of a sequence, started from ``initial_state`` (``(N, H, E, M)``
    float32, or ``None`` for zeros) and returning ``(product, final_state)``:

        S_l = initial_state + sum_{j<=l} keys_j values_j^T ;  product_l = S_l^T queries_l

    ``final_state`` is the ``S_i`` that the reference's step-wise attention keeps
    (``recurrent/attention/self_attention/linear_attention.py:63-90``), so a prompt processed
    here can be continued there, or by another call on the next piece.  Forward only (no
    autograd); enqueued on the current stream."""
    lib = _native.load()
    q, k, v = (_prepare(t, n) for t, n in
               ((queries, "queries"), (keys, "keys"), (values, "values")))
    N, H, L, E = q.shape
    M = v.shape[3]
    s0 = None
    if initial_state is not None:
        s0 = _prepare(initial_state, "initial_state")
        if s0.dtype != torch.float32 or tuple(s0.shape) != (N, H, E, M):
            raise RuntimeError("causal_dot_product_with_state: initial_state must be a float32 "
                               "tensor of shape (N, H, E, M)")
    out = torch.empty((N, H, L, M), dtype=torch.float32, device=q.device)
    s1 = torch.empty((N, H, E, M), dtype=torch.float32, device=q.device) if return_state else None
    with _device_guard(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = _workspace_bytes("ftc_causal_dot_product_workspace_bytes", N, H, L, E, M,
                                  _native.dtype_code(q.dtype))
        ws, nbytes = _workspace(nbytes, q.device, stream)
        dq, dk, dv, do = (_native.describe(t) for t in (q, k, v, out))
        d0 = _native.describe(s0) if s0 is not None else None
        d1 = _native.describe(s1) if s1 is not None else None
        rc = lib.ftc_causal_dot_product_state(dq, dk, dv, d0, do, d1,
                                              ws.data_ptr() if ws is not None else None, nbytes,
                                              stream)
        _native.check(rc, "ftc_causal_dot_product_state")
        _after_call(ws, stream)
    return out, s1


def causal_dot_backward_hip(queries, keys, values, grad_out, grad_queries, grad_keys,
                            grad_values):
    """In-place backward; replaces the reference's native ``causal_dot_backward``
    (``causal_product_cuda.cu:1438-1467``).  A gradient passed as ``None`` is skipped.
    Enqueued on the current stream."""
    lib = _native.load()
    q, k, v, g = (_prepare(t, n) for t, n in
                  ((queries, "queries"), (keys, "keys"), (values, "values"),
                   (grad_out, "grad_out")))
    if g.dtype != torch.float32:
        g = g.float()
    gq, gk, gv = (_check_out(t, n) if t is not None else None for t, n in
                  ((grad_queries, "grad_queries"), (grad_keys, "grad_keys"),
                   (grad_values, "grad_values")))
    N, H, L, E = q.shape
    M = v.shape[3]
    with _device_guard(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = _workspace_bytes("ftc_causal_dot_backward_workspace_bytes", N, H, L, E, M,
                                  _native.dtype_code(q.dtype))
        ws, nbytes = _workspace(nbytes, q.device, stream)
        descs = [_native.describe(t) if t is not None else None for t in (q, k, v, g, gq, gk, gv)]
        rc = lib.ftc_causal_dot_backward(*descs, ws.data_ptr() if ws is not None else None,
                                         nbytes, stream)
        _native.check(rc, "ftc_causal_dot_backward")
        _after_call(ws, stream)


FTC_ERR_UNSUPPORTED = -2


def fused_attention_covers(queries, values, keys=None):
    """True when ``ftc_causal_linear_attention`` has a kernel for tensors of these sizes and
    element type ((N, H, L, E) queries and keys, (N, H, L, M) values)."""
    tensors = (queries, values) if keys is None else (queries, keys, values)
    if any(t.dtype != torch.float32 or t.device != queries.device for t in tensors):
        return False
    if queries.device.type != "cuda":
        return False
    if keys is not None and keys.shape[3] != queries.shape[3]:
        return False
    return queries.shape[3] in (32, 64) and values.shape[3] in (32, 64)


def _check_key_lengths(key_lengths, q):
    if key_lengths is not None:
        if key_lengths.dtype != torch.int64 or key_lengths.device != q.device or \
                key_lengths.shape != (q.shape[0],) or not key_lengths.is_contiguous():
            raise RuntimeError("causal_linear_attention: key_lengths must be a contiguous int64 "
                               "tensor of N values on the device of the queries")


def causal_linear_attention_hip(queries, keys, values, key_lengths, eps, out, denominators=None):
    """In-place fused forward of causally masked linear attention with the feature map
    ``elu(x) + 1``: replaces the body of the reference module's forward
    (``attention/causal_linear_attention.py:71-104``) in one launch.  ``queries``, ``keys``:
    raw (N, H, L, E) projections; ``values``, ``out``: (N, H, L, M); ``key_lengths``: int64
    tensor of N lengths on the same device, or None; ``denominators``: None, or a float32
    (N, H, L) tensor that receives the normaliser's denominators (the backward needs them).
    Raises ``RuntimeError`` for sizes without a fused kernel (see ``fused_attention_covers``)."""
    lib = _native.load()
    q, k, v = (_prepare(t, n) for t, n in
               ((queries, "queries"), (keys, "keys"), (values, "values")))
    o = _check_out(out, "out")
    N, H, L, E = q.shape
    M = v.shape[3]
    _check_key_lengths(key_lengths, q)
    with _device_guard(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = _workspace_bytes("ftc_causal_linear_attention_workspace_bytes", N, H, L, E, M,
                                  _native.dtype_code(q.dtype))
        ws, nbytes = _workspace(nbytes, q.device, stream)
        dq, dk, dv, do = (_native.describe(t) for t in (q, k, v, o))
        dden = _native.describe(denominators.unsqueeze(3)) if denominators is not None else None
        rc = lib.ftc_causal_linear_attention_forward(
            dq, dk, dv, key_lengths.data_ptr() if key_lengths is not None else None, float(eps),
            do, dden, ws.data_ptr() if ws is not None else None, nbytes, stream)
        _native.check(rc, "ftc_causal_linear_attention_forward")
        _after_call(ws, stream)


def causal_linear_attention_backward_hip(queries, keys, values, key_lengths, out, denominators,
                                         grad_out, grad_queries, grad_keys, grad_values):
    """In-place backward of ``causal_linear_attention_hip``: gradients with respect to the raw
    queries, keys and values (any of the three may be None) from ``grad_out``, the forward's
    ``out`` and its ``denominators``.  Replaces what autograd does in the reference for the body
    of ``CausalLinearAttention.forward`` (``attention/causal_linear_attention.py:71-104``)."""
    lib = _native.load()
    q, k, v, o, g = (_prepare(t, n) for t, n in
                     ((queries, "queries"), (keys, "keys"), (values, "values"), (out, "out"),
                      (grad_out, "grad_out")))
    gq, gk, gv = (_check_out(t, n) if t is not None else None for t, n in
                  ((grad_queries, "grad_queries"), (grad_keys, "grad_keys"),
                   (grad_values, "grad_values")))
    N, H, L, E = q.shape
    M = v.shape[3]
    _check_key_lengths(key_lengths, q)
    with _device_guard(q.device):
        stream = torch.cuda.current_stream().cuda_stream
        nbytes = _workspace_bytes("ftc_causal_linear_attention_backward_workspace_bytes", N, H, L,
                                  E, M, _native.dtype_code(q.dtype))
        ws, nbytes = _workspace(nbytes, q.device, stream)
        descs = [_native.describe(t) if t is not None else None
                 for t in (q, k, v, o, denominators.unsqueeze(3), g, gq, gk, gv)]
        rc = lib.ftc_causal_linear_attention_backward(
            descs[0], descs[1], descs[2],
            key_lengths.data_ptr() if key_lengths is not None else None, *descs[3:],
            ws.data_ptr() if ws is not None else None, nbytes, stream)
        _native.check(rc, "ftc_causal_linear_attention_backward")
        _after_call(ws, stream)


class CausalLinearAttentionFunction(torch.autograd.Function):
    """``out = causal linear attention(queries, keys, values)`` with the feature map
    ``elu(x) + 1``, the key-length mask and the normaliser inside, one fused launch forward
    and one launch sequence backward.  Tensors in the operator's (N, H, L, X) layout (permuted
    views of the module's (N, L, H, X) tensors are fine)."""

    @staticmethod
    def forward(ctx, queries, keys, values, key_lengths, eps):
        N, H, L, _ = queries.shape
        M = values.shape[3]
        # (N, L, H, M) storage, as the module hands its result on
        out = torch.empty((N, L, H, M), device=queries.device, dtype=torch.float32).permute(0, 2, 1, 3)
        den = torch.empty((N, H, L), device=queries.device, dtype=torch.float32)
        causal_linear_attention_hip(queries, keys, values, key_lengths, eps, out, den)
        ctx.save_for_backward(queries, keys, values, out, den)
        ctx.key_lengths = key_lengths
        return out

    @staticmethod
    def backward(ctx, grad_out):
        queries, keys, values, out, den = ctx.saved_tensors
        need = ctx.needs_input_grad
        like = lambda t: torch.empty_like(t.permute(0, 2, 1, 3)).permute(0, 2, 1, 3)
        gq = like(queries) if need[0] else None
        gk = like(keys) if need[1] else None
        gv = like(values) if need[2] else None
        causal_linear_attention_backward_hip(queries, keys, values, ctx.key_lengths, out, den,
                                             grad_out, gq, gk, gv)
        return gq, gk, gv, None, None


def _cpu_args(name, *tensors):
    for t in tensors:
        if t.dim() != 4 or t.device.type != "cpu":
            raise RuntimeError("%s: expected 4-dimensional CPU tensors" % name)


def _cpu_scan(a, b, v, out, reverse, chunk=128):
    """out[l] = sum_{j<=l} (a_l . b_j) v_j on CPU tensors (reverse: j >= l), chunked along L:
    a running (D, F) state plus the masked product inside a chunk, float32 accumulation,
    written into ``out`` in place.  This is the package's own host path for CPU tensors (the
    reference keeps a ``"cpu"`` entry next to ``"cuda"``, ``__init__.py:23-30``); it shares
    nothing with the GPU path and is not a fallback for it."""
    N, H, L, D = a.shape
    state = a.new_zeros((N, H, D, v.shape[3]), dtype=torch.float32)
    starts = list(range(0, L, chunk))
    for lo in (reversed(starts) if reverse else starts):
        hi = min(L, lo + chunk)
        ac, bc, vc = (t[:, :, lo:hi].float() for t in (a, b, v))
        p = torch.matmul(ac, bc.transpose(2, 3))
        p = torch.triu(p) if reverse else torch.tril(p)
        out[:, :, lo:hi] = (torch.matmul(p, vc) + torch.matmul(ac, state)).to(out.dtype)
        state = state + torch.matmul(bc.transpose(2, 3), vc)


def causal_dot_product_cpu(queries, keys, values, product):
    """In-place forward for CPU tensors, the reference's native signature
    (``causal_product_cpu.cpp:82-87``)."""
    _cpu_args("causal_dot_product", queries, keys, values, product)
    _cpu_scan(queries, keys, values, product, False)


def causal_dot_backward_cpu(queries, keys, values, grad_out, grad_queries, grad_keys,
                            grad_values):
    """In-place backward for CPU tensors (``causal_product_cpu.cpp:133-141``): the three
    gradients are the same scan under a change of roles."""
    _cpu_args("causal_dot_backward", queries, keys, values, grad_out)
    if grad_queries is not None:
        _cpu_scan(grad_out, values, keys, grad_queries, False)
    if grad_keys is not None:
        _cpu_scan(values, grad_out, queries, grad_keys, True)
    if grad_values is not None:
        _cpu_scan(keys, queries, grad_out, grad_values, True)


class CausalDotProduct(torch.autograd.Function):
    """Compute the weighted sum of values but attending only to previous values
    (reference ``__init__.py:20-74``)."""
    dot = {
        "cpu": causal_dot_product_cpu,
        "cuda": causal_dot_product_hip,
    }
    dot_backward = {
        "cpu": causal_dot_backward_cpu,
        "cuda": causal_dot_backward_hip,
    }

    @staticmethod
    def forward(ctx, Q, K, V):
        ctx.save_for_backward(Q, K, V)

        device = Q.device
        N, H, L, _ = Q.shape
        _, _, _, M = V.shape
        # the kernels overwrite every element, so no zero fill is needed
        product = torch.empty((N, H, L, M), device=device, dtype=torch.float32)

        CausalDotProduct.dot[device.type](
            Q.data,
            K.data,
            V.data,
            product
        )
        return product

    @staticmethod
    def backward(ctx, grad_out):
        Q, K, V = ctx.saved_tensors

        grad_Q = torch.empty_like(Q, memory_format=torch.contiguous_format)
        grad_K = torch.empty_like(K, memory_format=torch.contiguous_format)
        grad_V = torch.empty_like(V, memory_format=torch.contiguous_format)

        CausalDotProduct.dot_backward[Q.device.type](
            Q.data,
            K.data,
            V.data,
            grad_out,
            grad_Q,
            grad_K,
            grad_V
        )
        return grad_Q, grad_K, grad_V


# Alias the autograd functions to python style snake case naming
causal_dot_product = CausalDotProduct.apply
