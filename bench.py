#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only c2,c3,c4,c5,next,sib] [--no-cpu-baseline]

The defaults (40 warm-up + 100 timed launches) are long enough for the GPU's clocks to settle under load; a
handful of launches reads ~15 % low.  A "step" is one launch of the FP8 GEMM at the headline configuration (M=N=K=8192, e4m3 operands,
B column-major, per-tensor fp32 scales, bf16 output) with inputs resident in HBM.  The JSON line also
carries the other three configurations (decode-shape GEMM, FP8 attention, MoE grouped GEMM) under
"other_workloads" together with the kernels either side of them (casts, quantisation, routing), each with its own roofline
object, and the ref-eager CPU path (ATen's CPU
torch._scaled_mm on the 1024^3 configuration) under "cpu_baseline".
"""
from __future__ import annotations

import argparse
import json
import os
import pathlib
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_FP8_TFLOPS = 5000.0   # MI355X dense FP8 MFMA
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense BF16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E


def _time_launches(fn, steps, warmup):
    """Average device time per call (ms) from HIP events on the launch stream, plus the wall-clock
    time of the same region bracketed by synchronisations."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(end) / steps, wall_ms


def _traffic(name):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE, scaled by a copy of known
    size), read from the `traffic_bytes <name> <bytes>` lines of the summary recorded under profiles/."""
    f = ROOT / "profiles" / "hbm_traffic_fetch_write_size.txt"
    if f.exists():
        for line in f.read_text().splitlines():
            parts = line.split()
            if len(parts) == 3 and parts[0] == "traffic_bytes" and parts[1] == name:
                return int(parts[2])
    return None


def bench_c2(steps, warmup):
    import torch
    import helion_amd as hx
    from helion_amd import inputs

    a, b, sa, sb = inputs.gemm_c2("cuda")
    fn = lambda: hx.fp8_gemm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
    ms, wall = _time_launches(fn, steps, warmup)
    flops = 2.0 * 8192**3
    tf = flops / (ms * 1e-3) / 1e12
    return ms, wall, {
        "bound": "mfma", "achieved": tf, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s", "frac": tf / PEAK_FP8_TFLOPS,
        "traffic": _traffic("fp8_gemm_tile256_c2"), "kernel": "hx_fp8_gemm_tile256", "avg_launch_ms": ms,
        "algorithmic_flops_per_launch": flops,
    }


def bench_c3(steps, warmup):
    import torch
    import helion_amd as hx
    from helion_amd import inputs

    a, b, sa, sb = inputs.gemm_c3("cuda")
    # the 224 MiB weight matrix fits the 256 MB Infinity Cache: rotate 6 distinct copies so every launch
    # streams its weights from HBM
    nbuf = 6
    bs = [b] + [b.T.contiguous().clone().T for _ in range(nbuf - 1)]
    state = {"i": 0}

    def fn():
        state["i"] = (state["i"] + 1) % nbuf
        return hx.fp8_gemm(a, bs[state["i"]], scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)

    ms, wall = _time_launches(fn, max(steps, 24), max(warmup, 12))
    m, n, k = 16, 28672, 8192
    nbytes = float(n * k + m * k + 2 * m * n)
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {
        "workload": "C3 decode fp8_gemm M16 N28672 K8192 bf16 out, 6 rotating weight buffers (HBM-cold)",
        "ms_per_launch": ms, "value": gbs, "unit": "GB/s",
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                     "traffic": _traffic("fp8_gemm_skinny_c3"), "kernel": "hx_fp8_gemm_skinny_direct", "avg_launch_ms": ms,
                     "algorithmic_bytes_per_launch": nbytes},
    }


def bench_c4(steps, warmup):
    import torch
    import helion_amd as hx
    from helion_amd import inputs

    q, k, v = inputs.attention_c4("cuda")
    flops = 4.0 * 4 * 32 * 4096 * 4096 * 128
    out = {}
    for mode, exact in (("exact_max", True), ("online", False)):
        fn = lambda: hx.fp8_attention_kernel(q, k, v, 4, 32, out_dtype=torch.float32, exact_max=exact)
        ms, wall = _time_launches(fn, min(steps, 50), min(warmup, 25))
        tf = flops / (ms * 1e-3) / 1e12
        out[mode] = {"ms_per_launch": ms, "tflops_counted": tf, "frac_fp8_peak": tf / PEAK_FP8_TFLOPS}
    tf = out["exact_max"]["tflops_counted"]
    return {
        "workload": "C4 fp8_attention B4 H32 S4096 D128 non-causal, fp32 out; flops counted as 4*B*H*S^2*D",
        "ms_per_launch": out["exact_max"]["ms_per_launch"], "value": tf, "unit": "TFLOP/s", "modes": out,
        "roofline": {"bound": "mfma", "achieved": tf, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s", "frac": tf / PEAK_FP8_TFLOPS,
                     "traffic": _traffic("fp8_attention_c4"), "kernel": "hx_fp8_attention_kernel<128,f32,exact>",
                     "avg_launch_ms": out["exact_max"]["ms_per_launch"], "algorithmic_flops_per_launch": flops},
    }


def bench_c5(steps, warmup):
    import torch
    import helion_amd as hx
    from helion_amd import inputs

    A, W, ex = inputs.moe_c5("cuda")
    args = hx.moe_matmul_ogs_helion_kernel_args_gen(A, W, ex)
    fn = lambda: hx.moe_matmul_ogs(*args)
    ms, wall = _time_launches(fn, min(steps, 30), min(warmup, 10))
    flops = 2.0 * 32768 * 4096 * 14336
    tf = flops / (ms * 1e-3) / 1e12
    return {
        "workload": "C5 moe_matmul_ogs 16384 tokens x top-2 (Zipf 1.2), K4096 N14336 E8 bf16",
        "ms_per_launch": ms, "value": tf, "unit": "TFLOP/s",
        "roofline": {"bound": "mfma", "achieved": tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tf / PEAK_BF16_TFLOPS,
                     "traffic": _traffic("moe_tile256_c5"), "kernel": "hx_gemm16_tile256<bf16, grouped> (+prep/mark/zero_rows)",
                     "avg_launch_ms": ms, "algorithmic_flops_per_launch": flops},
    }


def bench_next_rows(steps, warmup):
    """The kernels either side of the three hot kernels (routing tables, top-k entry, casts, quantisation), each against the
    HBM roofline of its algorithmic bytes.  Launch-latency-sized kernels are reported in microseconds as well."""
    import torch
    import helion_amd as hx
    from helion_amd import inputs

    out = {}
    n_it, n_w = min(steps, 50), min(warmup, 20)

    def hbm(nbytes, ms, kernel, workload):
        gbs = nbytes / (ms * 1e-3) / 1e9
        return {"workload": workload, "ms_per_launch": ms, "value": gbs, "unit": "GB/s",
                "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                             "traffic": None, "kernel": kernel, "avg_launch_ms": ms, "algorithmic_bytes_per_launch": float(nbytes)}}

    # preprocessing casts at the C4 shape: 3 x (fp16 in + e4m3 out)
    q, k, v = (torch.randn(4, 32, 4096, 128, device="cuda").to(torch.float16) for _ in range(3))
    ms, _ = _time_launches(lambda: hx.preprocess_fp8_attention_inputs(q, k, v), n_it, n_w)
    out["attention_preprocess_cast"] = hbm(3 * q.numel() * 3, ms, "hx_cast_e4m3_kernel<f16> x3 in one launch",
                                           "preprocess_fp8_attention_inputs at C4 shape, fp16 -> e4m3, 3 x 67M elements")
    del q, k, v
    # per-tensor quantisation of a bf16 8192^2 operand: read for amax, read again + write e4m3
    x = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    ms, _ = _time_launches(lambda: hx.fp8_quantize_per_tensor(x), n_it, n_w)
    out["fp8_quantize_per_tensor"] = hbm(x.numel() * 5, ms, "hx_amax_partial + hx_amax_final + hx_cast_e4m3_kernel<bf16>",
                                         "amax -> scale -> e4m3 of a bf16 8192x8192 operand (bytes: 2 reads + 1 write)")
    del x
    # a decode batch of 64 rows against the C3 weight matrix: the 128-column tile kernel as a weight-streaming loop
    bufs = [(torch.randn(28672, 8192, device="cuda") * 0.5).to(torch.float8_e4m3fn).T for _ in range(4)]
    xa = (torch.randn(64, 8192, device="cuda") * 0.5).to(torch.float8_e4m3fn)
    turn = [0]

    def decode64():
        turn[0] = (turn[0] + 1) % len(bufs)
        return hx.fp8_gemm(xa, bufs[turn[0]], out_dtype=torch.bfloat16)

    ms, _ = _time_launches(decode64, n_it, n_w)
    out["decode_gemm_m64"] = hbm(28672 * 8192 + 64 * 8192 + 2 * 64 * 28672, ms, "hx_fp8_gemm_tileN128<bf16, 64 rows, paired DMA>",
                                 "fp8_gemm M64 N28672 K8192 bf16 out, 4 rotating weight buffers (HBM-cold)")
    del bufs, xa
    # routing tables at the C5 row count and at 1M rows
    _, _, ex = inputs.moe_c5("cuda")
    ms, _ = _time_launches(lambda: hx.moe_routing(ex, 8), n_it, n_w)
    out["moe_routing_c5"] = hbm(ex.numel() * (8 + 8 + 4), ms, "hx_moe_routing_kernel<int64, one workgroup>",
                                "stable sort/count/scan of 32768 int64 expert ids, E=8 (launch-latency sized: see ms_per_launch)")
    big = ex.repeat(32)
    ms, _ = _time_launches(lambda: hx.moe_routing(big, 8), n_it, n_w)
    out["moe_routing_1m"] = hbm(big.numel() * (8 + 8 + 4), ms, "hx_moe_routing_kernel count + scan + scatter",
                                "the same for 1048576 rows (three launches)")
    return out


def bench_siblings(steps, warmup):
    """The 16-bit siblings (dense matmul with epilogue, split-K matmul, flash attention) at the fp8 configurations'
    shapes, against the bf16 MFMA roofline (split-K: launch-latency sized, reported in microseconds as well)."""
    import torch
    import helion_amd as hx
    from helion_amd.matmul import bias_relu

    out = {}
    n_it, n_w = min(steps, 30), min(warmup, 10)

    def mfma(flops, ms, kernel, workload, traffic=None):
        tf = flops / (ms * 1e-3) / 1e12
        return {"workload": workload, "ms_per_launch": ms, "value": tf, "unit": "TFLOP/s",
                "roofline": {"bound": "mfma", "achieved": tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tf / PEAK_BF16_TFLOPS,
                             "traffic": traffic, "kernel": kernel, "avg_launch_ms": ms, "algorithmic_flops_per_launch": float(flops)}}

    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(8192, 8192, device="cuda", generator=g).to(torch.bfloat16)
    y = torch.randn(8192, 8192, device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randn(8192, device="cuda", generator=g).to(torch.bfloat16)
    ep = bias_relu(bias)
    ms, _ = _time_launches(lambda: hx.matmul(x, y, ep), n_it, n_w)
    out["matmul_bf16_bias_relu"] = mfma(2.0 * 8192**3, ms, "hx_gemm16_tile256<bf16, dense + epilogue>",
                                        "matmul 8192^3 bf16, relu(acc + bias) fused, row-major operands", _traffic("gemm16_dense_8192"))
    del x, y, bias
    x = torch.randn(64, 32768, device="cuda", generator=g).to(torch.float16)
    y = torch.randn(32768, 64, device="cuda", generator=g).to(torch.float16)
    ms, _ = _time_launches(lambda: hx.matmul_split_k(x, y), n_it, n_w)
    out["matmul_split_k_fp16"] = mfma(2.0 * 64 * 64 * 32768, ms, "hx_gemm16_tile128<f16, split-K partials> + hx_matmul16_reduce",
                                      "matmul_split_k 64 x 32768 x 64 fp16 (the example's shape; launch-latency sized)")
    del x, y
    for d in (128, 64):
        q, k, v = (torch.randn(4, 32, 4096, d, device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
        ms, _ = _time_launches(lambda: hx.attention(q, k, v), n_it, n_w)
        out[f"attention_bf16_d{d}"] = mfma(4.0 * 4 * 32 * 4096 * 4096 * d, ms, f"hx_attention16_kernel<{d}, bf16>",
                                           f"attention B4 H32 S4096 D{d} bf16 non-causal; flops counted as 4*B*H*S^2*D", _traffic(f"attention16_d{d}"))
        del q, k, v
    return out


def cpu_baseline():
    """The reference's ref-eager CPU path for fp8_gemm (ATen CPU torch._scaled_mm, unit scales, fp32
    accumulate, bf16 result) on the 1024^3 configuration, repeated for about 10 s of CPU time."""
    import torch
    from helion_amd import inputs
    from oracle import oracle as orc

    a, b = inputs.gemm_c1()
    orc.fp8_gemm_ref_eager(a, b, torch.bfloat16)
    times = []
    t_end = time.perf_counter() + 10.0
    while time.perf_counter() < t_end and len(times) < 2000:
        t0 = time.perf_counter()
        orc.fp8_gemm_ref_eager(a, b, torch.bfloat16)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {
        "value": 2.0 * 1024**3 / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"fp8_gemm 1024x1024x1024 (config C1), ref-eager form on host CPU, median of {len(times)} runs (~10 s)",
        "seconds_per_run": med, "host_cpus": os.cpu_count(),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--only", default="c2,c3,c4,c5,next,sib")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run three plain 1 GiB device copies (a known-traffic kernel to scale rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (no sharding, no collectives); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback", file=sys.stderr)
        sys.exit(1)
    only = set(args.only.split(","))
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    ms, wall, roof = bench_c2(args.steps, args.warmup)
    others = {}
    if "c3" in only:
        others["c3_decode_gemm"] = bench_c3(args.steps, args.warmup)
        torch.cuda.empty_cache()
    if "c4" in only:
        others["c4_fp8_attention"] = bench_c4(args.steps, args.warmup)
        torch.cuda.empty_cache()
    if "c5" in only:
        others["c5_moe_grouped_gemm"] = bench_c5(args.steps, args.warmup)
        torch.cuda.empty_cache()
    if "next" in only:
        others.update(bench_next_rows(args.steps, args.warmup))
        torch.cuda.empty_cache()
    if "sib" in only:
        others.update(bench_siblings(args.steps, args.warmup))
        torch.cuda.empty_cache()
    line = {
        "metric": "FP8 GEMM/attention TFLOP/s + % of MI355X FP8 MFMA peak (or % HBM BW), 1 GPU",
        "value": roof["achieved"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {"workload": "C2 fp8_gemm M=N=K=8192, e4m3 A row-major x B column-major, per-tensor fp32 scales, "
                               "fp32 accumulate, bf16 out", "device": torch.cuda.get_device_name(0)},
        "roofline": roof,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(),
        "other_workloads": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
