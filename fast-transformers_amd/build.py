"""Compile the gfx950 causal-product library (hipcc, in-tree).

    python fast-transformers_amd/build.py [--force] [--verbose]

Output: fast_transformers_amd/libftc_causal.so next to the Python package, where
``fast_transformers_amd._native`` loads it.  hipcc cross-compiles, so no GPU is needed.
"""
import argparse
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OUT = os.path.join(HERE, "fast_transformers_amd", "libftc_causal.so")
OBJ_DIR = os.path.join(HERE, "build")

# -packed-fp32-ops is switched off on purpose: the compiler must not form
# v_pk_{add,mul,fma}_f32 from scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I", INCLUDE, "-I", CSRC,
]


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def headers():
    return sorted(glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(INCLUDE, "*.h")))


def build(force=False, verbose=False, extra_flags=()):
    hipcc = find_hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    newest_header = max(os.path.getmtime(h) for h in headers())
    objs = []
    procs = []
    for src in sources():
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        objs.append(obj)
        fresh = (os.path.exists(obj) and os.path.getmtime(obj) >= os.path.getmtime(src)
                 and os.path.getmtime(obj) >= newest_header)
        if fresh and not force:
            continue
        cmd = [hipcc, "-c", src, "-o", obj] + HIPCC_FLAGS + list(extra_flags)
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd)))
    for src, p in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on %s" % src)
    if procs or force or not os.path.exists(OUT):
        cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", OUT] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--verbose", action="store_true")
    a = ap.parse_args()
    print(build(force=a.force, verbose=a.verbose))
