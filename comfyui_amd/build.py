"""Compile comfyui_amd/csrc/*.hip into comfyui_amd/libhdmoe.so for gfx950 with hipcc.

hipcc cross-compiles without a GPU present. Run as `python -m comfyui_amd.build`
(or through __graft_entry__.build()). The library is built in-tree so that the
Python side can load it with ctypes from a fixed place.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhdmoe.so")
PROBE_LIB = os.path.join(HERE, "libhdmoe_probe.so")
SOURCES = ["gate.hip", "dispatch.hip", "elementwise.hip", "gemm.hip", "layer.hip", "weights.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # never let the compiler form packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(verbose=True, extra_flags=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if out and verbose:
            print(out)
        if p.returncode != 0:
            failed = True
            print(f"FAILED: {src}", file=sys.stderr)
            if not verbose:
                print(out, file=sys.stderr)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # an unresolved symbol (e.g. a kernel stub the host pass dropped) must fail the build, not the first call
    subprocess.check_call([sys.executable, "-c", f"import ctypes; ctypes.CDLL({LIB!r})"])
    # measurement support for bench.py --aux-kernels (the matrix cores' own rate); not part of the product library
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-shared", "-o", PROBE_LIB, os.path.join(CSRC, "mfma_probe.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        print(out.stdout, file=sys.stderr)
        raise RuntimeError("hipcc failed: mfma_probe.hip")
    return LIB


if __name__ == "__main__":
    build()
