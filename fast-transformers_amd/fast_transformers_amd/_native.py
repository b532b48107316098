"""ctypes binding of ``libftc_causal.so`` (C ABI: ``include/ftc_causal_product.h``).

No torch types cross the boundary: tensors are described by ``ftc_tensor4`` (device
pointer, dtype code, sizes and strides in elements), the stream is a raw
``hipStream_t`` and scratch memory is a raw device pointer the caller owns.

There is no fallback: when the library is missing, ``load()`` raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libftc_causal.so")

FTC_F32 = 0
FTC_BF16 = 1
_DTYPE_CODE = {torch.float32: FTC_F32, torch.bfloat16: FTC_BF16}

EXPORTED_SYMBOLS = (
    "ftc_version",
    "ftc_last_error",
    "ftc_last_kernel",
    "ftc_tuning_reload",
    "ftc_causal_dot_plan",
    "ftc_workspace_reset",
    "ftc_causal_dot_product_workspace_bytes",
    "ftc_causal_dot_product",
    "ftc_causal_dot_product_static",
    "ftc_causal_dot_product_state",
    "ftc_causal_dot_backward_workspace_bytes",
    "ftc_causal_dot_backward",
    "ftc_causal_linear_attention_workspace_bytes",
    "ftc_causal_linear_attention",
    "ftc_causal_linear_attention_forward",
    "ftc_causal_linear_attention_backward_workspace_bytes",
    "ftc_causal_linear_attention_backward",
)


class Tensor4(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("size", ctypes.c_int64 * 4),
        ("stride", ctypes.c_int64 * 4),
    ]


_lib = None


def load():
    """Load the HIP library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "fast_transformers_amd: %s is missing; build it with "
            "`python fast-transformers_amd/build.py` (there is no CPU or PyTorch fallback)"
            % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    t4 = ctypes.POINTER(Tensor4)
    lib.ftc_version.restype = ctypes.c_int
    lib.ftc_version.argtypes = []
    lib.ftc_last_error.restype = ctypes.c_char_p
    lib.ftc_last_error.argtypes = []
    lib.ftc_last_kernel.restype = ctypes.c_char_p
    lib.ftc_last_kernel.argtypes = []
    lib.ftc_tuning_reload.restype = ctypes.c_int
    lib.ftc_tuning_reload.argtypes = []
    for name in ("ftc_causal_dot_product_workspace_bytes",
                 "ftc_causal_dot_backward_workspace_bytes",
                 "ftc_causal_linear_attention_workspace_bytes",
                 "ftc_causal_linear_attention_backward_workspace_bytes"):
        f = getattr(lib, name)
        f.restype = ctypes.c_int64
        f.argtypes = [ctypes.c_int64] * 5 + [ctypes.c_int32]
    lib.ftc_workspace_reset.restype = ctypes.c_int
    lib.ftc_workspace_reset.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.ftc_causal_dot_product.restype = ctypes.c_int
    lib.ftc_causal_dot_product.argtypes = [t4] * 4 + [ctypes.c_void_p, ctypes.c_size_t,
                                                      ctypes.c_void_p]
    lib.ftc_causal_dot_product_static.restype = ctypes.c_int
    lib.ftc_causal_dot_product_static.argtypes = [t4] * 4 + [ctypes.c_void_p]
    lib.ftc_causal_dot_product_state.restype = ctypes.c_int
    lib.ftc_causal_dot_product_state.argtypes = [t4] * 6 + [ctypes.c_void_p, ctypes.c_size_t,
                                                            ctypes.c_void_p]
    lib.ftc_causal_dot_backward.restype = ctypes.c_int
    lib.ftc_causal_dot_backward.argtypes = [t4] * 7 + [ctypes.c_void_p, ctypes.c_size_t,
                                                       ctypes.c_void_p]
    lib.ftc_causal_linear_attention.restype = ctypes.c_int
    lib.ftc_causal_linear_attention.argtypes = [t4] * 3 + [ctypes.c_void_p, ctypes.c_float, t4,
                                                           ctypes.c_void_p, ctypes.c_size_t,
                                                           ctypes.c_void_p]
    lib.ftc_causal_linear_attention_forward.restype = ctypes.c_int
    lib.ftc_causal_linear_attention_forward.argtypes = [t4] * 3 + [ctypes.c_void_p, ctypes.c_float, t4,
                                                                   t4, ctypes.c_void_p,
                                                                   ctypes.c_size_t, ctypes.c_void_p]
    lib.ftc_causal_linear_attention_backward.restype = ctypes.c_int
    lib.ftc_causal_linear_attention_backward.argtypes = [t4] * 3 + [ctypes.c_void_p] + [t4] * 6 + [
        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.ftc_causal_dot_plan.restype = ctypes.c_int
    lib.ftc_causal_dot_plan.argtypes = [t4] * 3 + [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    _lib = lib
    return lib


def plan(shape_q, shape_v, dtype=FTC_F32, backward=False, strides=None):
    """Text of ``ftc_causal_dot_plan`` for dense (N, H, L, E) queries and keys and (N, H, L, M)
    values (or the element strides given as three 4-tuples): what the planner would launch.
    Needs no GPU."""
    def dense(shape, stride):
        d = Tensor4()
        d.ptr = None
        d.dtype = dtype
        st = stride or (shape[1] * shape[2] * shape[3], shape[2] * shape[3], shape[3], 1)
        for i in range(4):
            d.size[i], d.stride[i] = shape[i], st[i]
        return d
    st = strides or (None, None, None)
    q, k, v = dense(shape_q, st[0]), dense(shape_q, st[1]), dense(shape_v, st[2])
    buf = ctypes.create_string_buffer(16384)
    rc = load().ftc_causal_dot_plan(ctypes.byref(q), ctypes.byref(k), ctypes.byref(v),
                                    1 if backward else 0, buf, len(buf))
    check(rc, "ftc_causal_dot_plan")
    return buf.value.decode()


def last_error():
    return load().ftc_last_error().decode("utf-8", "replace")


def check(rc, what):
    if rc < 0:
        raise RuntimeError("%s failed (status %d): %s" % (what, rc, last_error()))
    return rc


def dtype_code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError("causal_dot_product: expected float32 or bfloat16 tensors, got %s"
                           % dtype) from None


def describe(t):
    """``ftc_tensor4`` view of a 4-d device tensor (no copy)."""
    shape = t.shape
    empty = shape[0] == 0 or shape[1] == 0 or shape[2] == 0 or shape[3] == 0
    return Tensor4(None if empty else t.data_ptr(), dtype_code(t.dtype), tuple(shape), t.stride())
