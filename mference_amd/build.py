"""Builds libmfmoe.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmfmoe.so")
SOURCES = ["format.hip", "gemv.hip", "router.hip", "router_family.hip", "moe_decode.hip", "moe_fused.hip", "moe_prefill.hip", "api.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",
    # packed-FP32 instructions are switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter",
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, "-o", LIB, *[os.path.join(CSRC, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libmfmoe.so")
    if verbose and proc.stderr:
        sys.stderr.write(proc.stderr)
    build_microbench(verbose)
    return LIB


def build_microbench(verbose: bool = False) -> str:
    """The stand-alone issue-port measurement (csrc/microbench/issue_port.hip): a program of its own,
    not part of libmfmoe.so."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    src = os.path.join(CSRC, "microbench", "issue_port.hip")
    exe = os.path.join(CSRC, "microbench", "issue_port")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-o", exe, src]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building microbench/issue_port")
    return exe


if __name__ == "__main__":
    print(build(verbose=True))
