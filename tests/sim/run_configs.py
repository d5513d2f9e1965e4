"""The BASELINE configurations executed in the host execution model (tests/sim) against the oracle, at their real sizes
where the model finishes in minutes: a parity record that needs no GPU.

    python tests/sim/run_configs.py [--only c1,c2,c3,c4,c5,d64,d128,d256] [--c4-heads 2] [--c5-columns 512] [--features MASK]

  C1  fp8_gemm 1024^3 (the reference's own CPU case)                         whole output, bit for bit
  C2  fp8_gemm 8192^3, per-tensor scales, bf16 out (the headline kernel)     whole output (about ten minutes)
  C3  decode fp8_gemm M16 N28672 K8192                                       whole output
  C4  fp8_attention B4 H32 S4096 D128, fp32 out                              `--c4-heads` heads of the 128, all 4096 queries,
                                                                             exact mode vs ref-eager oracle, online mode vs
                                                                             the 64-key tiled oracle
  C5  moe_matmul_ogs 32768 rows x K4096, 8 experts (Zipf top-2 routing)      all rows and all experts with the real routing
                                                                             tables, the first `--c5-columns` of the 14336
                                                                             output columns (the kernel treats column tiles
                                                                             independently)

  D64 / D128 / D256  decode fp8_gemm M64 / M128 / M256 N28672 K8192           whole output

--features MASK switches opt-in kernel paths on (helion_amd.HX_FEATURE_*): C2 then runs on the persistent 256x256 kernel
(mask 8), C5 on the persistent grouped kernel (64), the decode rows on the kernel with separate A / B rings (16).

Every operand sits in a guarded buffer and the LDS access check is on, as in the tests.  Prints one line per
configuration; exit status 1 if any is out of tolerance.  Not part of the default test run (tests/test_sim_configs.py
runs C1 and reduced forms of the others)."""
from __future__ import annotations

import argparse
import pathlib
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

import torch  # noqa: E402

from helion_amd import inputs  # noqa: E402
from oracle import oracle as orc  # noqa: E402
from tests._util import attention_close, rel_err  # noqa: E402
from tests.sim import simlib, simops  # noqa: E402


def c1():
    a, b = inputs.gemm_c1()
    out = simops.fp8_gemm(a, b, None, None, torch.bfloat16)
    ref = orc.fp8_gemm_ref_eager(a, b, torch.bfloat16)
    same = torch.equal(out.view(torch.int16), ref.view(torch.int16))
    return same, f"bit-identical to the ref-eager oracle: {same}; max|err|/max|ref| {rel_err(out, ref):.2e}"


def _gemm(a, b, sa, sb, path):
    out = simops.fp8_gemm(a, b, sa, sb, torch.bfloat16, want_path=path)
    ref = orc.fp8_gemm(a, b, sa, sb, torch.bfloat16)
    e = rel_err(out, ref)
    # the model sums an MFMA exactly and the oracle sums in fp32, so a bf16 rounding boundary can fall either way
    diff = int((out.view(torch.int16) != ref.view(torch.int16)).sum())
    return e <= 1e-2, f"max|err|/max|ref| {e:.2e} (tolerance 2e-2); {diff} of {out.numel()} bf16 results differ by a rounding step"


FEATURES = 0


def c2():
    return _gemm(*inputs.gemm_c2(), path=7 if FEATURES & 8 else 1)


def decode(rows):
    a, b, sa, sb = inputs.gemm_scaled(rows, 28672, 8192, rows)
    return _gemm(a, b, sa, sb, path=8 if FEATURES & 16 else 5)


def c3():
    return _gemm(*inputs.gemm_c3(), path=2)


def c4(heads):
    q, k, v = inputs.attention_c4()
    pick = [0, 77, 5, 126, 33, 64, 99, 18][:heads] if heads <= 8 else list(range(min(heads, q.shape[0])))
    qs, ks, vs = (torch.stack([t[h] for h in pick]) for t in (q, k, v))
    ok, notes = True, []
    for exact in (True, False):
        out = simops.fp8_attention(qs, ks, vs, 1, len(pick), torch.float32, exact, "DS", want_path=1)
        ref = orc.fp8_attention(qs, ks, vs, 1, len(pick), torch.float32) if exact else orc.fp8_attention_tiled(qs, ks, vs, 1, len(pick), 64, torch.float32)
        good = attention_close(out, ref)
        ok &= good
        notes.append(f"{'exact-max vs ref-eager' if exact else 'online vs 64-key tiled'} oracle: max|err|/max|ref| {rel_err(out, ref):.2e} ({'ok' if good else 'OUT OF TOLERANCE'})")
    return ok, f"heads {pick if len(pick) <= 8 else 'all ' + str(len(pick))}: " + "; ".join(notes)


def c5(columns):
    A, W, ex = inputs.moe_c5()
    W = W[:, :, :columns].contiguous()
    E = W.shape[0]
    idx = torch.argsort(ex, stable=True).to(torch.int32)
    counts = torch.bincount(ex, minlength=E).to(torch.int32)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0)
    out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=6 if FEATURES & 64 else 3, poison=9.0)
    ref = orc.moe_matmul_ogs_reference(A, W, ex)
    e = rel_err(out, ref)
    return e <= 1e-2, f"rows per expert {counts.tolist()}, columns 0..{columns - 1}: max|err|/max|ref| {e:.2e} (tolerance 2e-2)"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", default="c1,c3,c4,c5,c2")
    ap.add_argument("--c4-heads", type=int, default=2)
    ap.add_argument("--c5-columns", type=int, default=512)
    ap.add_argument("--variant", default="lazy", choices=list(simlib.VARIANTS))
    ap.add_argument("--features", type=int, default=0)
    args = ap.parse_args()
    simlib.configure(args.variant)
    global FEATURES
    FEATURES = args.features
    simlib.load().hx_set_features(FEATURES)
    runs = {"c1": c1, "c2": c2, "c3": c3, "c4": lambda: c4(args.c4_heads), "c5": lambda: c5(args.c5_columns),
            "d64": lambda: decode(64), "d128": lambda: decode(128), "d256": lambda: decode(256)}
    bad = 0
    for name in args.only.split(","):
        t0 = time.time()
        simlib.work()
        ok, note = runs[name]()
        w = simlib.work()
        print(f"{name.upper()} {'ok ' if ok else 'BAD'} {note}  [{w['workgroups']} workgroups, {w['mfma']} wave-level MFMAs, "
              f"{w['dma_bytes'] / 2**20:.0f} MiB by DMA, {time.time() - t0:.0f} s, variant {args.variant}, features {FEATURES}]", flush=True)
        bad += not ok
    sys.exit(1 if bad else 0)


if __name__ == "__main__":
    main()
