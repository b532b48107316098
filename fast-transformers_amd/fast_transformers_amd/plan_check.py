"""Check the planner's choice of kernel against the forced alternatives on this GPU.

    python -m fast_transformers_amd.plan_check [--widths 64x64,32x128] [--dtype f32|bf16]
                                               [--chains 4,16,64,256,1024] [--lengths 256,...]
                                               [--margin 0.07] [--min-rows R] [--max-rows R] [--quick]

Which kernel runs a launch is decided on the host from the sizes alone (csrc/ftc_mfma.hip), by
rules whose thresholds were measured.  This tool measures them again: for every shape of the
sweep it times forward and backward as the planner routes them and under each setting of the
FTC_* tuning variables that forces another route, and prints the launches where a forced route
is more than ``--margin`` faster.  An empty list means the rules still hold on this GPU; a
region of neighbouring shapes in the list is a threshold to move.  Single lines of a few
percent on launches of 20 to 30 microseconds are run-to-run spread.

Needs the built library and a GPU; nothing here is used by the operator itself.
"""
import argparse
import os
import sys

# tuning variables that force a route (read by the library at first use and at reload_tuning())
MODES = {
    "planner": {},
    "kernels that split L": {"FTC_TP": "0", "FTC_TPX": "0"},
    "no exchange": {"FTC_TPX": "0"},
    "chain-parallel": {"FTC_TP": "1"},
}
FORCING = sorted({name for env in MODES.values() for name in env})
DEFAULT_WIDTHS = "64x64,128x128,32x128,128x32,64x128,32x32,96x96"


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--widths", default=DEFAULT_WIDTHS, help="ExM pairs, comma separated")
    ap.add_argument("--dtype", choices=("f32", "bf16"), default="f32",
                    help="element type of Q, K, V (the gradient of the product is fp32)")
    ap.add_argument("--chains", default="4,16,64,256,1024", help="values of N*H")
    ap.add_argument("--lengths", default="256,1024,4096,16384,65536", help="values of L")
    ap.add_argument("--margin", type=float, default=0.07)
    ap.add_argument("--max-rows", type=int, default=1 << 21, help="skip shapes with more chains * L")
    ap.add_argument("--min-rows", type=int, default=1 << 14, help="skip shapes with fewer chains * L")
    ap.add_argument("--quick", action="store_true", help="64x64 only, three chain counts")
    a = ap.parse_args(argv)
    if a.quick:
        a.widths, a.chains = "64x64", "8,80,512"
    a.widths = [tuple(int(x) for x in w.split("x")) for w in a.widths.split(",")]
    a.chains = [int(x) for x in a.chains.split(",")]
    a.lengths = [int(x) for x in a.lengths.split(",")]
    return a


def shapes(a):
    for E, M in a.widths:
        for chains in a.chains:
            for L in a.lengths:
                if a.min_rows <= chains * L <= a.max_rows:
                    yield E, M, chains, L


def main(argv=None):
    a = parse_args(argv)
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("plan_check needs a GPU")
    from . import _native, causal_product as cp

    saved = {name: os.environ.pop(name, None) for name in FORCING}
    dtype = torch.bfloat16 if a.dtype == "bf16" else torch.float32

    def timed(call):
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(10):
            call()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) * 100.0, _native.load().ftc_last_kernel().decode()

    # the clocks ramp over the first tenth of a second of work
    warm = torch.empty(1 << 26, device="cuda")
    for _ in range(200):
        warm.zero_()
    torch.cuda.synchronize()
    del warm

    wrong, count = [], 0
    try:
        for E, M, chains, L in shapes(a):
            q, k = (torch.randn(1, chains, L, E, device="cuda").to(dtype) for _ in range(2))
            v = torch.randn(1, chains, L, M, device="cuda").to(dtype)
            g = torch.randn(1, chains, L, M, device="cuda")
            out = torch.empty(1, chains, L, M, device="cuda")
            dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            calls = {"forward": lambda: cp.causal_dot_product_hip(q, k, v, out),
                     "backward": lambda: cp.causal_dot_backward_hip(q, k, v, g, dq, dk, dv)}
            for direction, call in calls.items():
                result = {}
                # (the planner's own route once more at the end: the first timing of a shape
                # also pays for its cold rows)
                for mode in list(MODES) + ["planner"]:
                    for name in FORCING:
                        os.environ.pop(name, None)
                    os.environ.update(MODES[mode])
                    cp.reload_tuning()
                    t = timed(call)
                    if mode not in result or t[0] < result[mode][0]:
                        result[mode] = t
                count += 1
                own, kernel = result["planner"]
                best = min((m for m in MODES if m != "planner"), key=lambda m: result[m][0])
                if result[best][0] < (1.0 - a.margin) * own:
                    wrong.append("%3d x %-3d %-4s %5d chains  L=%-6d %-8s planner %8.1f us (%s)   %s %8.1f us (%s)"
                                 % (E, M, a.dtype, chains, L, direction, own, kernel, best,
                                    result[best][0], result[best][1]))
                    print(wrong[-1], flush=True)
    finally:
        for name in FORCING:
            os.environ.pop(name, None)
        os.environ.update({n: v for n, v in saved.items() if v is not None})
        cp.reload_tuning()
    print("%d launches timed, %d with a forced route more than %.0f %% faster than the planner's"
          % (count, len(wrong), 100 * a.margin))
    return 0


if __name__ == "__main__":
    sys.exit(main())
