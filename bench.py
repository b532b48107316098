#!/usr/bin/env python3
"""Benchmark of the causal linear-attention product on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg5|cfg4op|cfg4|wide]

A step is one forward + backward of ``causal_dot_product`` over one batch of synthetic input,
called through the C ABI with outputs and workspace pre-allocated and every input already in
HBM.  The default workload is the configuration the metric is quoted on:
N=10, H=8, L=1000, E=M=64, fp32.  Steps rotate over several input sets (> 512 MB in total) so
that the 256 MB Infinity Cache cannot serve a step from the previous one.

Prints ONE JSON line.  ``value`` is N*L / t(fwd+bwd) in Mtokens/s.  ``roofline`` is the mean
over the two launches of a step (forward: one scan, backward: three scans side by side):
algorithmic bytes per launch = 4*((2E+2M) + (4E+3M))/2 per (n,h,l) position for fp32 (forward
reads Q,K,V and writes the product; backward reads Q,K,V,G and writes dQ,dK,dV), algorithmic
flops 14*E*M/2, over the mean of the two launch durations, timed with events on the stream
the kernels are launched on; both the HBM and the matrix-core fraction are given and the one
with the larger minimum time is named as the bound.  With the default workload the line also
carries a few timed steps of cfg3 and cfg5 and of the attention module's training step at
config 4's attention shape (``config.secondary``).  ``cpu_baseline`` times
the reference's own CPU extension (or, when it is not built, its C restatement) on this box's
host cores over a bounded number of calls of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "fast-transformers_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix, published

# HBM-side bytes per scan-kernel launch (mean of the forward and the backward launch) from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, scaled by what the same
# counters read for the 256 MiB copy of --calibrate-copy; the runs are summarised in
# profiles/*_<workload>_traffic.md.  Each figure is stamped with the hash of
# the kernel sources it was measured with (kernel_source_hash() below): the JSON line
# carries it only while the sources are unchanged, otherwise null.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {
    # workload: (bytes, kernel source hash at the time of the measurement)
    "cfg2": (139695660, "58af0cd3d23348b6"),
    "cfg3": (2610208921, "58af0cd3d23348b6"),
    "cfg5": (4976938155, "58af0cd3d23348b6"),
    "wide": (1877438021, "58af0cd3d23348b6"),
}

WORKLOADS = {
    # name: (N, H, L, E, M, dtype, seed)
    "cfg2": (10, 8, 1000, 64, 64, "f32", 2),
    "cfg3": (1, 16, 65536, 64, 64, "f32", 3),
    "cfg4op": (10, 8, 4096, 64, 64, "f32", 4),
    "cfg5": (4, 32, 16384, 32, 128, "bf16", 5),
    # not one of the reference's configurations: a 128 x 128 state, for the profiles of the
    # chain-parallel kernel's wide form
    "wide": (8, 16, 4096, 128, 128, "f32", 6),
}


def kernel_source_hash():
    """First 16 hex digits of the SHA-256 over the kernel sources (csrc/*.h, *.hip) and the
    C ABI header, in name order."""
    import glob
    import hashlib
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(ROOT, "fast-transformers_amd", "csrc", "*.h*")) +
                       glob.glob(os.path.join(ROOT, "include", "*.h"))):
        h.update(os.path.basename(path).encode())
        h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    entry = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(workload)
    if entry is None or entry[1] != kernel_source_hash():
        return None
    return entry[0]


def alg_bytes_per_position(E, M, dtype):
    """(forward, backward) algorithmic bytes per (n,h,l) position."""
    if dtype == "f32":
        return 4 * (2 * E + 2 * M), 4 * (4 * E + 3 * M)
    # bf16 Q,K,V and their gradients; product and upstream gradient fp32
    return 2 * (2 * E + M) + 4 * M, 2 * (2 * E + M) + 4 * M + 2 * (2 * E + M)


def measure(workload, steps, warmup, ramp_ms, sets_arg=0, calibrate_copy=False, wrapper_leg=True):
    """Times `steps` forward + backward steps of one workload through the C ABI and returns the
    JSON line's dictionary (without the CPU baseline)."""
    import torch
    from fast_transformers_amd import _native
    from fast_transformers_amd.causal_product import causal_dot_product_hip, \
        causal_dot_backward_hip
    dev = torch.device("cuda:0")
    N, H, L, E, M, dtype, seed = WORKLOADS[workload]
    tdtype = torch.float32 if dtype == "f32" else torch.bfloat16
    esz = 4 if dtype == "f32" else 2
    set_bytes = N * H * L * ((2 * E + M) * esz * 2 + 2 * M * 4)
    nsets = sets_arg or max(1, min(8, -(-(768 << 20) // set_bytes)))

    gen = torch.Generator(device="cpu").manual_seed(seed)
    sets = []
    for s in range(nsets):
        if s == 0:
            import torch.nn.functional as F
            Q = F.elu(torch.randn(N, H, L, E, generator=gen)) + 1
            K = F.elu(torch.randn(N, H, L, E, generator=gen)) + 1
            V = torch.randn(N, H, L, M, generator=gen)
            G = torch.randn(N, H, L, M, generator=gen)
            base = [Q.to(tdtype).to(dev), K.to(tdtype).to(dev), V.to(tdtype).to(dev), G.to(dev)]
            ins = base
        else:
            # further sets: same distribution, decorrelated by a roll along L (device-side)
            ins = [torch.roll(t, shifts=17 * s, dims=2).contiguous() for t in base]
        outs = [torch.empty(N, H, L, M, device=dev, dtype=torch.float32),
                torch.empty(N, H, L, E, device=dev, dtype=tdtype),
                torch.empty(N, H, L, E, device=dev, dtype=tdtype),
                torch.empty(N, H, L, M, device=dev, dtype=tdtype)]
        sets.append((ins, outs))

    # The timed path is the C ABI itself: descriptors, workspace and stream are prepared
    # once, a step is two library calls (the Python wrapper's per-call cost is reported
    # separately as wrapper_overhead_us).
    import ctypes
    lib = _native.load()
    code = _native.dtype_code(tdtype)
    ws_bytes = max(lib.ftc_causal_dot_product_workspace_bytes(N, H, L, E, M, code),
                   lib.ftc_causal_dot_backward_workspace_bytes(N, H, L, E, M, code))
    assert ws_bytes >= 0, _native.last_error()
    ws = torch.zeros(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    ws_ptr = ctypes.c_void_p(ws.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    keep_alive = [[_native.describe(t) for t in ins + outs] for ins, outs in sets]
    descs = [[ctypes.byref(d) for d in row] for row in keep_alive]

    def fwd(i):
        q, k, v, g, o, dq, dk, dv = descs[i % nsets]
        rc = lib.ftc_causal_dot_product(q, k, v, o, ws_ptr, ws_bytes, stream)
        if rc:
            raise RuntimeError(_native.last_error())

    def bwd(i):
        q, k, v, g, o, dq, dk, dv = descs[i % nsets]
        rc = lib.ftc_causal_dot_backward(q, k, v, g, dq, dk, dv, ws_ptr, ws_bytes, stream)
        if rc:
            raise RuntimeError(_native.last_error())

    def step(i):
        fwd(i)
        bwd(i)

    if calibrate_copy:
        src = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # which kernels the planner picks for this workload
    fwd(0)
    fwd_kernel = lib.ftc_last_kernel().decode()
    bwd(0)
    bwd_kernel = lib.ftc_last_kernel().decode()

    # set-up: a fresh GPU takes a few hundred milliseconds of load to reach its clocks
    t_ramp = time.perf_counter()
    i = 0
    while (time.perf_counter() - t_ramp) * 1e3 < ramp_ms:
        for _ in range(20):
            step(i)
            i += 1
        torch.cuda.synchronize()
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps

    # per-direction device time with events on the launch stream
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for i in range(steps):
        ev[i][0].record()
        fwd(i)
        ev[i][1].record()
        bwd(i)
        ev[i][2].record()
    torch.cuda.synchronize()
    assert int(ws[8:12].view(torch.int32).item()) == 0, "a wavefront gave up waiting"

    # cost of going through the Python wrapper instead (same work, wall clock)
    wrapper_ms = float("nan")
    if wrapper_leg:
        for i in range(5):   # (first use: the wrapper's own workspace and pinned probe word)
            (q, k, v, g), (o, dq, dk, dv) = sets[i % nsets]
            causal_dot_product_hip(q, k, v, o)
            causal_dot_backward_hip(q, k, v, g, dq, dk, dv)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for i in range(steps):
            (q, k, v, g), (o, dq, dk, dv) = sets[i % nsets]
            causal_dot_product_hip(q, k, v, o)
            causal_dot_backward_hip(q, k, v, g, dq, dk, dv)
        torch.cuda.synchronize()
        wrapper_ms = (time.perf_counter() - t2) * 1e3 / steps
    fwd_ms = sorted(e[0].elapsed_time(e[1]) for e in ev)
    bwd_ms = sorted(e[1].elapsed_time(e[2]) for e in ev)
    fwd_avg, bwd_avg = sum(fwd_ms) / len(fwd_ms), sum(bwd_ms) / len(bwd_ms)

    TH = N * H * L
    fb, bb = alg_bytes_per_position(E, M, dtype)
    bwd_gbps = bb * TH / (bwd_avg * 1e-3) / 1e9
    fwd_gbps = fb * TH / (fwd_avg * 1e-3) / 1e9
    value = N * L / (ms_per_step * 1e-3) / 1e6
    # The dominant kernel is the scan kernel: with E = M one step launches it twice (forward:
    # one scan; backward: three scans side by side).  Its roofline entry averages over those
    # two launches: algorithmic bytes per launch = (fwd + bwd bytes) / 2, duration = mean of
    # the two event-timed launches.
    launch_ms = (fwd_avg + bwd_avg) / 2
    launch_bytes = (fb + bb) * TH / 2
    launch_gbps = launch_bytes / (launch_ms * 1e-3) / 1e9
    # Both rooflines for the same launch.  Algorithmic flops are those of the recurrence,
    # 14 E M per position for forward + backward; for fp32 rows they are priced against the
    # fp32 matrix peak, for bf16 rows against the bf16 one.  The binding roofline is the one
    # with the larger minimum time.
    launch_flops = 14 * E * M * TH / 2
    mfma_peak = MFMA_FP32_PEAK_TFLOPS if dtype == "f32" else MFMA_BF16_PEAK_TFLOPS
    launch_tflops = launch_flops / (launch_ms * 1e-3) / 1e12
    t_hbm, t_mfma = launch_bytes / (HBM_PEAK_GBPS * 1e9), launch_flops / (mfma_peak * 1e12)
    hbm_entry = {"achieved": round(launch_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                 "frac": round(launch_gbps / HBM_PEAK_GBPS, 4)}
    mfma_entry = {"achieved": round(launch_tflops, 2), "peak": mfma_peak, "unit": "TFLOP/s",
                  "frac": round(launch_tflops / mfma_peak, 4)}
    bound = "mfma" if t_mfma > t_hbm else "hbm"
    binding = mfma_entry if bound == "mfma" else hbm_entry

    result = {
        "metric": "causal_dot_product fwd+bwd Mtokens/s (H=8,E=M=64); % of HBM/MFMA roofline",
        "value": round(value, 3),
        "unit": "Mtokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if dtype == "f32" else "bf16 in / f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "%s: causal_dot_product fwd+bwd N=%d H=%d L=%d E=%d M=%d %s"
                               % (workload, N, H, L, E, M, dtype),
                   "input_sets_rotated": nsets,
                   "token_heads_per_s": round(TH / (ms_per_step * 1e-3), 1),
                   "python_wrapper_ms_per_step": round(wrapper_ms, 5),
                   "fwd_ms_avg": round(fwd_avg, 5), "fwd_ms_min": round(fwd_ms[0], 5),
                   "bwd_ms_avg": round(bwd_avg, 5), "bwd_ms_min": round(bwd_ms[0], 5),
                   "fwd_alg_GBps": round(fwd_gbps, 1),
                   "fwdbwd_alg_GBps": round((fb + bb) * TH / (ms_per_step * 1e-3) / 1e9, 1),
                   "fwdbwd_alg_TFLOPs": round(14 * E * M * TH / (ms_per_step * 1e-3) / 1e12, 2),
                   "fwdbwd_frac_of_hbm_roofline":
                       round((fb + bb) * TH / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
        "roofline": {"bound": bound,
                     "kernel": "forward: %s, backward: %s (mean over the two launches)"
                               % (fwd_kernel, bwd_kernel),
                     "achieved": binding["achieved"], "peak": binding["peak"],
                     "unit": binding["unit"], "frac": binding["frac"],
                     "hbm": hbm_entry, "mfma": mfma_entry,
                     "min_time_us": {"hbm": round(t_hbm * 1e6, 2), "mfma": round(t_mfma * 1e6, 2)},
                     "launch_ms_avg": round(launch_ms, 5),
                     "alg_bytes_per_launch": int(launch_bytes),
                     "alg_flops_per_launch": int(launch_flops),
                     "traffic": measured_traffic(workload),
                     "kernel_source_hash": kernel_source_hash()},
    }

    return result, (N, H, L, E, M, seed)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: 1000; 50 for cfg4)")
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps first (default: 200, past the clock ramp; 5 for cfg4)")
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS) + ["cfg4"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-secondary", action="store_true",
                    help="cfg2 only: skip the few timed steps of cfg3 and cfg5 that the line "
                         "carries as config.secondary")
    ap.add_argument("--sets", type=int, default=0, help="input sets to rotate over (0 = auto)")
    ap.add_argument("--ramp-ms", type=float, default=300.0,
                    help="set-up: untimed steps for this many milliseconds before the warm-up "
                         "steps, so that the GPU clocks have ramped (0 to skip)")
    ap.add_argument("--print-kernel-hash", action="store_true",
                    help="print the kernel source hash that stamps measured traffic and exit")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device copy (a known-size kernel for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.steps is None:
        args.steps = 50 if args.workload == "cfg4" else 1000
    if args.warmup is None:
        args.warmup = 5 if args.workload == "cfg4" else 200
    if args.print_kernel_hash:
        print(kernel_source_hash())
        return
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path shards over N*H with no "
              "communication; no multi-GPU figure is produced). Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from fast_transformers_amd import _native
    from fast_transformers_amd.causal_product import causal_dot_product_hip, \
        causal_dot_backward_hip

    if args.workload == "cfg4":
        return encoder_workload(args)

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    _native.load()
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")

    result, (N, H, L, E, M, seed) = measure(args.workload, args.steps, args.warmup, args.ramp_ms,
                                            args.sets, args.calibrate_copy)
    # The other two single-kernel configurations, a few steps each, in the same line: the
    # long-sequence shape (cfg3) and the bf16 / asymmetric one (cfg5).
    if args.workload == "cfg2" and not args.no_secondary:
        torch.cuda.empty_cache()
        secondary = {}
        for name in ("cfg3", "cfg5"):
            r, _ = measure(name, 10, 3, 100.0, wrapper_leg=False)
            secondary[name] = {
                "workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"],
                "Mtokens_per_s": r["value"], "fwd_ms_avg": r["config"]["fwd_ms_avg"],
                "bwd_ms_avg": r["config"]["bwd_ms_avg"], "bound": r["roofline"]["bound"],
                "hbm_frac": r["roofline"]["hbm"]["frac"], "mfma_frac": r["roofline"]["mfma"]["frac"],
                "kernels": r["roofline"]["kernel"], "steps": 10, "warmup": 3, "ramp_ms": 100}
            torch.cuda.empty_cache()
        secondary["cfg4_attention_training"] = attention_training_step()
        result["config"]["secondary"] = secondary
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(N, H, L, E, M, seed, args.workload)
    print(json.dumps(result))


def attention_training_step(steps=10, warmup=3):
    """Forward + backward of the CausalLinearAttention module on the attention shape of
    config 4 (N=10, L=4096, 8 heads, E=M=64, fp32): through the fused entry points (one launch
    forward; element-wise pass, three scans and prefix-sum pass backward) and through the
    composition of operator calls that autograd differentiates piece by piece.  Wall clock
    over `steps` calls after `warmup`, inputs resident."""
    import torch
    from fast_transformers_amd import attention, masking
    from fast_transformers_amd.attention import causal_linear_attention as cla

    N, L, H, E, M = 10, 4096, 8, 64, 64
    gen = torch.Generator(device="cuda").manual_seed(4)
    q, k, v, w = (torch.randn(N, L, H, d, device="cuda", generator=gen) for d in (E, E, M, M))
    lengths = masking.LengthMask(torch.full((N,), L, device="cuda"), max_len=L)
    mask = masking.TriangularCausalMask(L, device="cuda")
    module = attention.CausalLinearAttention(E).cuda()

    def step():
        leaves = [t.detach().requires_grad_(True) for t in (q, k, v)]
        module(*leaves, mask, lengths, lengths).backward(w)

    def timed():
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    fused_ms = timed()
    covers = cla.fused_attention_covers
    cla.fused_attention_covers = lambda *a, **kw: False
    try:
        composed_ms = timed()
    finally:
        cla.fused_attention_covers = covers
    return {"workload": "CausalLinearAttention forward + backward, N=10 L=4096 H=8 E=M=64 fp32",
            "fused_ms_per_step": round(fused_ms, 4), "composition_ms_per_step": round(composed_ms, 4),
            "fused_Mtokens_per_s": round(N * L / (fused_ms * 1e-3) / 1e6, 2),
            "steps": steps, "warmup": warmup}


def encoder_workload(args):
    """Config 4: eval forward of an 8-layer causal-linear encoder (8 heads, query/value
    dims 64, d_model 512, FFN 1024, random-init weights) on rand(10, 4096, 512).  A step is
    one forward pass; the share of causal_dot_product is timed with events around the
    native call inside the attention module."""
    import torch
    from fast_transformers_amd.attention import build_causal_linear_encoder
    from fast_transformers_amd.attention import causal_linear_attention as cla
    from fast_transformers_amd.masking import TriangularCausalMask

    torch.cuda.set_device(0)
    torch.manual_seed(4)
    N, L, D = 10, 4096, 512
    enc = build_causal_linear_encoder(8, 8, 64, 64, 1024).cuda().eval()
    x = torch.rand(N, L, D, generator=torch.Generator().manual_seed(4)).cuda()
    mask = TriangularCausalMask(L, device="cuda")
    op_events = []
    # the native entry points the attention module may call: the fused one (feature map,
    # mask, product and normaliser in one launch) when it covers the sizes, else the product
    natives = {name: getattr(cla, name)
               for name in ("causal_linear_attention_hip", "causal_dot_product_hip")}
    used = set()

    def timed(name):
        def call(*a):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            natives[name](*a)
            e1.record()
            op_events.append((e0, e1))
            used.add(name)
        return call

    with torch.no_grad():
        t_ramp = time.perf_counter()
        while (time.perf_counter() - t_ramp) * 1e3 < args.ramp_ms:
            enc(x, attn_mask=mask)
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            enc(x, attn_mask=mask)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            enc(x, attn_mask=mask)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        for name in natives:
            setattr(cla, name, timed(name))
        for _ in range(args.steps):
            enc(x, attn_mask=mask)
        torch.cuda.synchronize()
        for name in natives:
            setattr(cla, name, natives[name])
    op_ms = sum(a.elapsed_time(b) for a, b in op_events) / args.steps
    fused = used == {"causal_linear_attention_hip"}
    # The events above bracket the Python wrapper, so when the GPU has run dry they also see
    # the host preparing the call.  The launch itself: the same native entry on the
    # encoder's (N, L, H, 64) layout, back to back over rotating inputs (> 512 MB, cold).
    with torch.no_grad():
        gen = torch.Generator(device="cuda").manual_seed(4)
        sets = [[torch.randn(N, L, 8, 64, device="cuda", generator=gen) for _ in range(3)]
                + [torch.empty(N, L, 8, 64, device="cuda")] for _ in range(3)]
        nhl = lambda t: t.permute(0, 2, 1, 3)

        def launch(i):
            q, k, v, o = sets[i % 3]
            if fused:
                natives["causal_linear_attention_hip"](nhl(q), nhl(k), nhl(v), None, 1e-6, nhl(o))
            else:
                natives["causal_dot_product_hip"](nhl(q), nhl(k), nhl(v), nhl(o))
        for i in range(10):
            launch(i)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(60):
            launch(i)
        e1.record()
        torch.cuda.synchronize()
        launch_ms = e0.elapsed_time(e1) / 60
        del sets
    TH = N * 8 * L
    # roofline of the operator's launches inside the encoder (8 per forward pass, one per
    # layer): forward only, so 4 E M flops and (2E + 2M) * 4 bytes per position; the fused
    # launch also carries the normaliser (4 E flops more) and reads and writes the same rows
    fb, _ = alg_bytes_per_position(64, 64, "f32")
    launch_bytes, launch_flops = fb * TH, 4 * 64 * (64 + (1 if fused else 0)) * TH
    gbps = launch_bytes / (launch_ms * 1e-3) / 1e9
    tflops = launch_flops / (launch_ms * 1e-3) / 1e12
    t_hbm = launch_bytes / (HBM_PEAK_GBPS * 1e9)
    t_mfma = launch_flops / (MFMA_FP32_PEAK_TFLOPS * 1e12)
    hbm_entry = {"achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                 "frac": round(gbps / HBM_PEAK_GBPS, 4)}
    mfma_entry = {"achieved": round(tflops, 2), "peak": MFMA_FP32_PEAK_TFLOPS,
                  "unit": "TFLOP/s", "frac": round(tflops / MFMA_FP32_PEAK_TFLOPS, 4)}
    bound = "mfma" if t_mfma > t_hbm else "hbm"
    binding = mfma_entry if bound == "mfma" else hbm_entry
    result = {
        "metric": "causal-linear encoder eval forward Mtokens/s (8 layers, d_model 512); "
                  "share of the native attention launches reported in config",
        "value": round(N * L / (ms * 1e-3) / 1e6, 3), "unit": "Mtokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cfg4: 8-layer causal-linear TransformerEncoder eval forward, "
                               "X=rand(10,4096,512), 8 heads, E=M=64, FFN 1024",
                   "native_entry": sorted(used),
                   "native_launch_ms": round(launch_ms, 5),
                   "native_share_of_forward": round(8 * launch_ms / ms, 4),
                   "native_ms_per_forward_bracketed_in_model": round(op_ms, 4),
                   "causal_dot_product_fwd_alg_GBps": round(gbps, 1)},
        "roofline": {"bound": bound,
                     "kernel": ("scan_wg_kernel<64,64,NORM> (ftc_causal_linear_attention" if fused
                                else "scan_dma_kernel (ftc_causal_dot_product")
                               + ": the operator's forward launch, one per layer; the rest of "
                                 "the encoder is torch's GEMMs and elementwise work)",
                     "achieved": binding["achieved"], "peak": binding["peak"],
                     "unit": binding["unit"], "frac": binding["frac"],
                     "hbm": hbm_entry, "mfma": mfma_entry,
                     "min_time_us": {"hbm": round(t_hbm * 1e6, 2), "mfma": round(t_mfma * 1e6, 2)},
                     "launch_ms_avg": round(launch_ms, 5),
                     "alg_bytes_per_launch": int(launch_bytes),
                     "alg_flops_per_launch": int(launch_flops),
                     "traffic": None,
                     "kernel_source_hash": kernel_source_hash()},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(N, 8, L, 64, 64, 4, "cfg4", forward_only=True)
    print(json.dumps(result))


def cpu_baseline(N, H, L, E, M, seed, workload, forward_only=False):
    """The reference's CPU extension (oracle/_ref) or its restatement, fwd+bwd, fp32, timed
    the way the reference's benchmark does (warm-up calls, then timed calls, wall clock;
    tests/causal_product/test_causal_product_cpu.py:87-99).  ``forward_only``: the
    operator's share of an eval forward pass (the encoder around it is not part of the
    checker), in tokens of one layer's call per second."""
    import torch
    import oracle
    Q, K, V, G = oracle.make_inputs(N, H, L, E, M, seed)
    out = torch.empty(N, H, L, M)
    gq, gk, gv = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    if oracle.reference_extension_available():
        ref = oracle.load_reference_extension()
        fwd, bwd, kind = ref.causal_dot_product, ref.causal_dot_backward, "reference"
    else:
        fwd, bwd, kind = oracle.causal_dot_product, oracle.causal_dot_backward, "port"

    def call():
        fwd(Q, K, V, out)
        if not forward_only:
            bwd(Q, K, V, G, gq, gk, gv)

    t = time.perf_counter()
    call()
    one = time.perf_counter() - t
    warm = 10 if one < 0.5 else 1
    timed = 10 if one < 0.5 else (3 if one < 5 else 1)
    for _ in range(warm):
        call()
    t = time.perf_counter()
    for _ in range(timed):
        call()
    dt = (time.perf_counter() - t) / timed
    threads = torch.get_num_threads()
    try:
        threads = int(os.environ.get("OMP_NUM_THREADS", "")) or threads
    except ValueError:
        pass
    return {"value": round(N * L / dt / 1e6, 4), "unit": "Mtokens/s",
            "cores": min(threads, N * H), "kind": kind,
            "sample": "%s %s fp32, %d warm-up + %d timed calls, %.1f ms per call; "
                      "OpenMP over N*H=%d chains, host cpu_count=%d"
                      % (workload,
                         "operator forward only (one layer's call)" if forward_only else "fwd+bwd",
                         warm, timed, dt * 1e3, N * H, os.cpu_count())}


if __name__ == "__main__":
    main()
