"""Builds libbgemm_mi355x.so for gfx950 with hipcc (no torch extension machinery)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SO = os.path.join(HERE, "libbgemm_mi355x.so")
SOURCES = ["api.hip", "pack.hip", "gemm_mfma.hip", "gemm_valu.hip", "gemm_skinny.hip", "gemm_chain.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         # "#pragma unroll" on loops with run-time bounds is a request, not a requirement
         "-Wno-pass-failed",
         # keep the compiler from forming packed-fp32 VALU ops
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for s in SOURCES:
        o = os.path.join(HERE, "build", s.replace(".hip", ".o"))
        objs.append(o)
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(CSRC, s), "-o", o]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((s, subprocess.Popen(cmd)))
    for s, p in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on %s" % s)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", SO] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return SO


def build_probes(root, verbose=True):
    """bench.py's measurement probes (bench_probes.hip beside it) -> libbench_probes.so, not part of the library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    so = os.path.join(root, "libbench_probes.so")
    cmd = [hipcc] + FLAGS + ["-shared", "-o", so, os.path.join(root, "bench_probes.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return so


if __name__ == "__main__":
    build()
    sys.stdout.write(SO + "\n")
