"""ftc_causal_dot_product_static (the entry point that allocates nothing) against
ftc_causal_dot_product on the same inputs, through the C ABI.

Both run the same kernels with the same segment plan and every sum has a fixed order, so
the two products must agree bit for bit.  The built-in scratch array keeps the previous
call's contents: the test makes two calls in a row, the second on a smaller input.
"""
import ctypes

import pytest
import torch

import oracle
from parity import scale_error

pytestmark = pytest.mark.gpu


def _call_pair(lib, native, shape, seed, dtype=torch.float32, check_memory=True):
    N, H, L, E, M = shape
    Q, K, V, _ = oracle.make_inputs(N, H, L, E, M, seed)
    Qd, Kd, Vd = (t.to(dtype).cuda() for t in (Q, K, V))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    descs = [native.describe(t) for t in (Qd, Kd, Vd)]

    # the existing entry point, with a caller-owned workspace
    want = torch.full((N, H, L, M), float("nan"), device="cuda")
    nbytes = native.check(
        lib.ftc_causal_dot_product_workspace_bytes(N, H, L, E, M, native.dtype_code(dtype)),
        "workspace_bytes")
    ws = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device="cuda")
    native.check(lib.ftc_causal_dot_product(*descs, native.describe(want), ws.data_ptr(), nbytes,
                                            stream), "ftc_causal_dot_product")

    # the entry point under test: outputs are allocated before the call, nothing inside it
    got = torch.full((N, H, L, M), float("nan"), device="cuda")
    torch.cuda.synchronize()
    # device memory as the driver sees it (not torch's cache): a hipMalloc inside the call,
    # by the library or anything it uses, would lower the free amount
    free_before, _ = torch.cuda.mem_get_info()
    allocs_before = torch.cuda.memory_stats().get("allocation.all.allocated", 0)
    native.check(lib.ftc_causal_dot_product_static(*descs, native.describe(got), stream),
                 "ftc_causal_dot_product_static")
    torch.cuda.synchronize()
    if check_memory:
        assert torch.cuda.mem_get_info()[0] >= free_before
        assert torch.cuda.memory_stats().get("allocation.all.allocated", 0) == allocs_before
    return Q, K, V, got.cpu(), want.cpu(), nbytes


def test_static_scratch_entry_point_matches_workspace_entry_point():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU")
    from fast_transformers_amd import _native as native
    lib = native.load()
    # first call: segments and a state exchange (scratch in use); second call: a smaller
    # input on the same array; third: bf16 rows; fourth: a shape of the generic path
    shapes = [((3, 4, 1500, 64, 64), 31, torch.float32),
              ((2, 3, 333, 64, 64), 32, torch.float32),
              ((2, 4, 2048, 32, 128), 33, torch.bfloat16),
              ((2, 2, 700, 25, 40), 34, torch.float32)]
    # set-up: the first call on a device makes the HIP runtime load the part of the library's
    # device code that holds the scratch array; later calls touch no allocator at all
    _call_pair(lib, native, (1, 2, 200, 64, 64), 30, check_memory=False)
    for shape, seed, dtype in shapes:
        print("static scratch", shape, dtype, flush=True)
        Q, K, V, got, want, nbytes = _call_pair(lib, native, shape, seed, dtype)
        assert nbytes > 0, "the case must use scratch memory"
        assert torch.isfinite(got).all()
        assert torch.equal(got, want)
        if dtype == torch.float32:
            assert scale_error(got, oracle.forward(Q, K, V)) <= 1e-4


def test_static_scratch_refuses_sizes_beyond_the_array():
    import os
    from fast_transformers_amd import _native as native
    lib = native.load()
    N, H, L, E, M = 4, 4, 65536, 500, 500  # odd widths: segment states of 1 MB each
    need = lib.ftc_causal_dot_product_workspace_bytes(N, H, L, E, M, native.FTC_F32)
    assert need > (48 << 20)
    # ... and so does the route without padded copies, which the entry point falls back to
    # before it gives up (asked of the host alone, with the copies switched off): only then is
    # it safe to hand the entry point descriptors whose pointers must never be read
    os.environ["FTC_PAD"] = "0"
    try:
        assert lib.ftc_tuning_reload() == 0
        bare = lib.ftc_causal_dot_product_workspace_bytes(N, H, L, E, M, native.FTC_F32)
    finally:
        del os.environ["FTC_PAD"]
        assert lib.ftc_tuning_reload() == 0
    assert bare > (48 << 20), "the sizes of this test no longer exceed the built-in array"
    # refused on the host before anything touches the device: the pointers are never read
    def fake(X):
        return native.Tensor4(256, native.FTC_F32, (N, H, L, X), (H * L * X, L * X, X, 1))
    q, k, v, o = fake(E), fake(E), fake(M), fake(M)
    rc = lib.ftc_causal_dot_product_static(ctypes.byref(q), ctypes.byref(k), ctypes.byref(v),
                                           ctypes.byref(o), None)
    assert rc == -3 and "scratch" in native.last_error()
