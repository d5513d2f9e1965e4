"""Distance check for the kernels that issue MFMAs as inline assembly (hx_mfma_*_acc / _overwrite, hx_acc_read in hx_common.h).

For inline assembly the compiler inserts neither the wait states between an MFMA and a vector instruction that reads its
result, nor those between a vector instruction that writes a register and an MFMA that reads it as a source operand.  The
persistent tile kernels are written so that neither pair ever comes close; this script compiles a source file for gfx950,
walks the generated code of the kernels named on the command line and reports the smallest distance, in instructions,
of (1) a v_accvgpr_read from the MFMA that wrote the register and (2) an MFMA from a vector-ALU write to one of its A / B
source registers.  Exit status 1 if either is below --min (default 24 instructions; the longest requirement of the
architecture is 18 wait states, and every instruction takes at least one).

    python helion_amd/csrc/scan_mfma_hazards.py fp8_gemm.hip hx_fp8_gemm_tile256p
    python helion_amd/csrc/scan_mfma_hazards.py moe_gemm.hip hx_gemm16_tile256p
    python helion_amd/csrc/scan_mfma_hazards.py matmul16.hip hx_gemm16_tile256p
"""
from __future__ import annotations

import argparse
import pathlib
import re
import subprocess
import sys
import tempfile

CSRC = pathlib.Path(__file__).resolve().parent
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _regs(tok: str):
    tok = tok.strip().rstrip(",")
    m = re.match(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return m.group(1), set(range(int(m.group(2)), int(m.group(3)) + 1))
    m = re.match(r"([va])(\d+)$", tok)
    if m:
        return m.group(1), {int(m.group(2))}
    return None, set()


def scan(asm: str, kernel: str, window: int):
    """[(mangled name, instructions, min distance MFMA -> accumulator read, min distance VALU write -> MFMA source)]"""
    out = []
    for m in re.finditer(r"^(_Z\w*%s\w*):" % re.escape(kernel), asm, re.M):
        body = asm[m.end():asm.index(".Lfunc_end", m.end())]
        ins = [ln.strip() for ln in body.split("\n") if ln.strip() and not ln.strip().startswith((";", "."))]
        d_read = d_src = window + 1
        for i, ln in enumerate(ins):
            if ln.startswith("v_mfma"):
                srcs = [_regs(o) for o in ln.split(None, 1)[1].split(",")[1:3]]
                for j in range(max(0, i - window), i):
                    p = ins[j]
                    if p.startswith("v_") and not p.startswith(("v_mfma", "v_cmp")):
                        k, d = _regs(p.split(None, 1)[1].split(",")[0])
                        if k == "v" and any(sk == "v" and d & sr for sk, sr in srcs):
                            d_src = min(d_src, i - j)
            elif ln.startswith("v_accvgpr_read"):
                _, src = _regs(ln.split(",")[1])
                for j in range(max(0, i - window), i):
                    p = ins[j]
                    if p.startswith("v_mfma"):
                        k, d = _regs(p.split(None, 1)[1].split(",")[0])
                        if k == "a" and d & src:
                            d_read = min(d_read, i - j)
        out.append((m.group(1), len(ins), d_read, d_src))
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("source")
    ap.add_argument("kernel")
    ap.add_argument("--min", type=int, default=24)
    args = ap.parse_args()
    with tempfile.TemporaryDirectory() as d:
        subprocess.run(["hipcc", *FLAGS, "-I", str(CSRC.parent.parent / "include"), "-c", str(CSRC / args.source), "-o", d + "/x.o", "-save-temps=obj"],
                       check=True, cwd=d, capture_output=True)
        asm = next(pathlib.Path(d).glob("*gfx950.s")).read_text()
    rows = scan(asm, args.kernel, 4 * args.min)
    if not rows:
        print(f"no kernel matching {args.kernel} in {args.source}")
        return 1
    bad = 0
    for name, n, d_read, d_src in rows:
        far = f"> {4 * args.min}"
        print(f"{name}: {n} instructions; accumulator read after its MFMA: {d_read if d_read <= 4 * args.min else far} instructions; "
              f"MFMA after a vector-ALU write to its source: {d_src if d_src <= 4 * args.min else far}")
        bad += d_read < args.min or d_src < args.min
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
