"""Builds libmfmoe.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmfmoe.so")
SOURCES = ["format.hip", "gemv.hip", "router.hip", "router_family.hip", "moe_decode.hip", "moe_fused.hip",
           "moe_prefill.hip", "static_scratch.hip", "api.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",
    # packed-FP32 instructions are switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter",
]


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed: " + " ".join(cmd[-3:]))
    if verbose and proc.stderr:
        sys.stderr.write(proc.stderr)


def build(verbose: bool = False, only: list[str] | None = None) -> str:
    """Compiles every source to an object of its own (in parallel) and links them.  `only` names the
    sources to recompile when the other objects are already there (a developer's shortcut; the build
    check compiles everything)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in SOURCES]
    if only is not None:
        only = [s if s.endswith(".hip") else s + ".hip" for s in only]
        unknown = [s for s in only if s not in SOURCES]
        if unknown:
            raise ValueError(f"not a source of the library: {unknown}")
    todo = [(s, o) for s, o in zip(SOURCES, objs) if only is None or s in only or not os.path.exists(o)]
    jobs = min(8, max(1, (os.cpu_count() or 2) // 2))
    with ThreadPoolExecutor(jobs) as pool:
        list(pool.map(lambda so: _run([hipcc, *FLAGS, "-c", "-o", so[1], os.path.join(CSRC, so[0])], verbose), todo))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, only=sys.argv[1:] or None))
