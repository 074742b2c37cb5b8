"""Build libdeltacnn_hip.so for gfx950 with hipcc (no GPU needed: cross-compiles).

    python deltacnn_amd/csrc/build.py [--force]

Objects land in deltacnn_amd/csrc/build/, the library in deltacnn_amd/.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "libdeltacnn_hip.so")
SOURCES = ["dc_abi.cpp", "elementwise.hip", "conv.hip", "convres.hip", "pwconv.hip", "pwpair.hip", "pool.hip", "block.hip", "linear.hip"]
HEADERS = ["common.hpp", "tile.hpp", "epilogue.hpp", os.path.join("..", "..", "include", "deltacnn_hip.h")]
# -ffp-contract=off: every operation of the bit-exact elementwise operators rounds on its own.
# packed-fp32-ops disabled: hipcc must not form v_pk_*_f32 from ordinary float code.
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    bdir = os.path.join(HERE, "build")
    os.makedirs(bdir, exist_ok=True)
    hdrs = [os.path.join(HERE, h) for h in HEADERS] + [os.path.abspath(__file__)]
    jobs = []
    objs = []
    for src in SOURCES:
        sp = os.path.join(HERE, src)
        obj = os.path.join(bdir, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        if force or _stale(obj, [sp] + hdrs):
            jobs.append([hipcc, "-x", "hip", *FLAGS, "-c", sp, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
        # the host pass does not know the device-only target feature; that line is harmless
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if err.strip():
            print(err, file=sys.stderr, flush=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed ({r.returncode}): {' '.join(cmd)}")

    with ThreadPoolExecutor(max_workers=min(4, max(1, len(jobs)))) as ex:
        list(ex.map(run, jobs))
    if force or jobs or _stale(LIB, objs):
        run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
