"""Builds tests/sim/libhx_sim.so: the kernel sources of helion_amd/csrc compiled for the host CPU against the execution
model in hx_sim.h / hx_sim.cpp, behind the same C ABI as the real library (test infrastructure: nothing under helion_amd/
refers to it).

    python tests/sim/build.py [-q]

The sources are copied into tests/sim/_build with two kinds of change, both listed here and nowhere else:
  * helion_amd/csrc/hx_common.h is replaced by tests/sim/hx_common.h (the same names; inline assembly and the launch
    helper expressed through the model);
  * the inline assembly inside the kernel files themselves (REWRITES below) is replaced by the C it stands for, and the
    one place where a kernel relies on the lanes of a wave executing an instruction together is marked as a wave-wide
    step.
Everything else is compiled exactly as the device compiler sees it."""
from __future__ import annotations

import hashlib
import pathlib
import re
import shutil
import subprocess
import sys

SIM = pathlib.Path(__file__).resolve().parent
ROOT = SIM.parent.parent
CSRC = ROOT / "helion_amd" / "csrc"
BUILD = SIM / "_build"
LIB = SIM / "libhx_sim.so"
CXX = "/opt/rocm/llvm/bin/clang++"
UNITS = ["hx_common.cpp", "fp8_gemm.hip", "fp8_attention.hip", "moe_gemm.hip", "moe_routing.hip", "fp8_quantize.hip",
         "matmul16.hip", "attention16.hip", "diag.hip"]
FLAGS = ["-std=c++17", "-O1", "-g", "-fPIC", "-fno-strict-aliasing", "-ffp-contract=off", "-Wno-unknown-attributes",
         "-Wno-unused-value", "-Wno-builtin-macro-redefined", "-Wno-reserved-macro-identifier", "-Wno-macro-redefined",
         "-Wno-ignored-attributes", "-Wno-pass-failed", "-Wno-unknown-pragmas", "-fno-stack-protector", "-mf16c"]

# (file, what the device source says, what the host build compiles instead)
REWRITES = [
    ("fp8_attention.hip", 'asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));', "d = fmaxf(fmaxf(a, b), c);"),
    ("fp8_attention.hip", 'asm volatile("" : "+v"(nv));', ";"),
    ("fp8_gemm.hip", 'asm volatile("" : "+v"(zero));', ";"),
    ("gemm16_tile256.h", 'asm volatile("" : "+v"(t));', ";"),
    # The lanes of a wave execute one instruction together: all of them have read the slot before the first lane of the
    # group stores the advanced one.  The model runs the lanes of a wave one after the other between two cross-lane
    # instructions, so the place where the kernel relies on that order is marked as one.
    ("moe_routing.hip", "    const int slot = hist[w][e];  // every lane of the group reads before its first lane advances the slot\n",
     "    const int slot = hist[w][e];\n    hxsim::wave_sync(__LINE__);\n"),
    # Pass 1 of the exact-max attention refills its K fragments after every round; after a wave's last tile the refill
    # re-reads that tile's slot, the values go unused, and by then pass 2's first DMA may already be writing the slot.  The
    # host build leaves that one read out, so that the LDS access check can stay strict everywhere else.
    ("fp8_attention.hip", "          kf[n] = load_kfrag(sk2, n);\n", "          if (more) kf[n] = load_kfrag(sk2, n);\n"),
    ("hx_common.cpp", "#include <hip/hip_runtime.h>", ""),
    ("hx_common.cpp", '#include "../../include/hx_kernels.h"', '#include "hx_kernels.h"'),
]


def _stamp() -> str:
    h = hashlib.sha256()
    for p in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h")) + list(CSRC.glob("*.cpp")) + list(SIM.glob("hx_*")) + [SIM / "selftest_kernels.cpp"]
                    + [SIM / "build.py", ROOT / "include" / "hx_kernels.h"]):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()


def is_current() -> bool:
    s = BUILD / "stamp"
    return LIB.exists() and s.exists() and s.read_text() == _stamp()


def build(verbose: bool = False, only_if_stale: bool = False) -> pathlib.Path:
    """Builds tests/sim/libhx_sim.so.  One build at a time: processes that find the library stale together (parallel test
    workers, two scripts started side by side) queue up on a lock file, and with only_if_stale the later ones find the work done."""
    import fcntl
    with open(SIM / ".build.lock", "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if only_if_stale and is_current():
            return LIB
        return _build_locked(verbose)


def _build_locked(verbose: bool) -> pathlib.Path:
    if BUILD.exists():
        shutil.rmtree(BUILD)
    BUILD.mkdir(parents=True)
    for p in list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h")) + list(CSRC.glob("*.cpp")):
        if p.name == "hx_common.h":
            continue
        text = p.read_text()
        for name, old, new in REWRITES:
            if name == p.name:
                if old not in text:
                    raise RuntimeError(f"{p.name}: the text a host rewrite applies to is gone: {old!r}")
                text = text.replace(old, new)
        if re.search(r"\basm\b", text):
            raise RuntimeError(f"{p.name}: inline assembly without a host rewrite")
        (BUILD / (p.name.replace(".hip", ".cpp") if p.suffix == ".hip" else p.name)).write_text(text)
    shutil.copy(SIM / "hx_common.h", BUILD / "hx_common.h")
    procs, objs = [], []
    # kernel objects: every load and store reports its address to the model (hx_sim.cpp: LDS access discipline)
    common = [CXX, *FLAGS, "-fsanitize-coverage=inline-8bit-counters,trace-loads,trace-stores", "-I", str(ROOT / "include"), "-I", str(SIM),
              "-include", str(SIM / "hx_sim.h")]
    for u in UNITS:
        src = BUILD / u.replace(".hip", ".cpp")
        obj = BUILD / (src.stem + ".o")
        cmd = [*common, "-c", str(src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd))
        procs.append((u, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(str(obj))
    shutil.copy(SIM / "selftest_kernels.cpp", BUILD / "selftest_kernels.cpp")
    obj = BUILD / "selftest_kernels.o"
    procs.append(("selftest_kernels.cpp", subprocess.Popen([*common, "-c", str(BUILD / "selftest_kernels.cpp"), "-o", str(obj)],
                                                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs.append(str(obj))
    obj = BUILD / "hx_sim.o"
    procs.append(("hx_sim.cpp", subprocess.Popen([CXX, *FLAGS, "-O3", "-I", str(SIM), "-c", str(SIM / "hx_sim.cpp"), "-o", str(obj)],
                                                 stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs.append(str(obj))
    for u, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f"host build of {u} failed:\n{out[-6000:]}")
        if verbose and out.strip():
            print(out)
    subprocess.check_call([CXX, "-shared", "-fPIC", "-o", str(LIB), *objs, "-ldl"])
    (BUILD / "stamp").write_text(_stamp())
    return LIB


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
