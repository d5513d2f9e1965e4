"""Builds helion_amd/libhx_kernels.so (gfx950 only) from helion_amd/csrc with hipcc.

    python -m helion_amd.build            # rebuild unconditionally
The shared object is built in-tree so it travels with the source tree; nothing is JIT-compiled
at import time and the Python layer refuses to run without it."""
from __future__ import annotations

import pathlib
import subprocess
import sys

PKG = pathlib.Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libhx_kernels.so"
SOURCES = ["hx_common.cpp", "fp8_gemm.hip", "fp8_attention.hip", "moe_gemm.hip", "moe_routing.hip", "fp8_quantize.hip",
           "matmul16.hip", "attention16.hip", "diag.hip"]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build(verbose: bool = False) -> pathlib.Path:
    objs = []
    procs = []
    for src in SOURCES:
        obj = CSRC / (src.rsplit(".", 1)[0] + ".o")
        cmd = ["hipcc", *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(str(obj))
    for src, p in procs:
        out, _ = p.communicate()
        filtered = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip() != "1 warning generated.")
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and filtered.strip():
            print(filtered)
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs])
    return LIB


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
