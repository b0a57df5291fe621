"""Compiles libiomx.so (HIP kernels + C ABI) and libiomx_probe.so (bandwidth probes and device
self-tests for the benchmark and the tests) for gfx950, in-tree.

    python -m iom_amd.build

The library is built into iom_amd/lib/ so that it travels with the source tree;
nothing is JIT-compiled at import time.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libiomx.so")
PROBE_LIB = os.path.join(LIBDIR, "libiomx_probe.so")

SOURCES = [
    "iomx_runtime.hip",
    "iomx_elementwise.hip",
    "iomx_rmsnorm.hip",
    "iomx_softmax.hip",
    "iomx_transfer.hip",
    "iomx_leaves.hip",
    "iomx_layer.hip",
    "iomx_linear.hip",
    "iomx_sdpa.hip",
]
# measurement and self-tests: a library of its own, so that libiomx.so exports operations and
# runtime only
PROBE_SOURCES = ["iomx_probe.hip"]

# -ffp-contract=off: no fused multiply-add may replace the reference's two
# roundings.  Packed FP32 instructions are disabled for the device pass.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def build_iomx(verbose: bool = True) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES + PROBE_SOURCES:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        cmd = [hipcc(), *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
               "-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    for src, proc in procs:
        out, _ = proc.communicate()
        text = "\n".join(l for l in out.decode().splitlines()
                         if "packed-fp32-ops" not in l and l.strip())
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if verbose and text:
            print(text)
    probe_objs = objs[len(SOURCES):]
    objs = objs[:len(SOURCES)]
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIB,
                           *probe_objs])
    objs += probe_objs
    for obj in objs:
        os.remove(obj)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build_iomx()
    sys.exit(0)
