"""Builds the C restatement (oracle/ref_c.c) into oracle/liboracle_c.so with gcc.
Test infrastructure only; the product library never links or loads it."""
from __future__ import annotations

import pathlib
import subprocess

HERE = pathlib.Path(__file__).resolve().parent
LIB = HERE / "liboracle_c.so"


def build(force: bool = True) -> pathlib.Path:
    src = HERE / "ref_c.c"
    if force or not LIB.exists() or LIB.stat().st_mtime < src.stat().st_mtime:
        subprocess.check_call(["gcc", "-O2", "-fPIC", "-shared", "-ffp-contract=off", "-o", str(LIB), str(src), "-lm"])
    return LIB


if __name__ == "__main__":
    print(build())
