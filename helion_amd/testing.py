"""The example harness the reference's scripts call (`helion._testing.run_example`, helion/_testing.py:341-404):
check every implementation against the first baseline in fp32 with `torch.testing.assert_close`, then time them all
and print a table to stderr.  Same argument names, defaults and tolerance convention."""
from __future__ import annotations

import sys
from typing import Callable

import torch


def do_bench(fn: Callable[[], object], warmup: int = 10, rep: int = 50) -> float:
    """Mean milliseconds per call from HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(rep):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / rep


def run_example(kernel_fn, baseline_fn, args: tuple, kernel_name: str = "helion_amd", baseline_name: str = "torch",
                rtol: float = 1e-2, atol: float = 1e-1) -> None:
    kernels = dict(kernel_fn) if isinstance(kernel_fn, dict) else {kernel_name: kernel_fn}
    baselines = dict(baseline_fn) if isinstance(baseline_fn, dict) else {baseline_name: baseline_fn}
    everything = {**kernels, **baselines}
    ref_name = next(iter(baselines))
    expected = baselines[ref_name](*args).to(torch.float32)
    for name, fn in everything.items():
        if name == ref_name:
            continue
        print(f"Testing {name} correctness...", file=sys.stderr)
        torch.testing.assert_close(fn(*args).to(torch.float32), expected, rtol=rtol, atol=atol)
    times = {name: do_bench(lambda fn=fn: fn(*args)) for name, fn in everything.items()}
    best = min(times[name] for name in baselines)
    bar = "=" * 65
    print(f"\n{bar}\nBenchmark Results\n{bar}", file=sys.stderr)
    print(f"{'Implementation':<20} {'Time (ms)':<12} {'Speedup':<15}\n{'-' * 65}", file=sys.stderr)
    for name, t in times.items():
        tag = "1.00x (ref)" if (name in baselines and t == best) else f"{best / t:.2f}x"
        print(f"{name:<20} {t:<12.4f} {tag:<15}", file=sys.stderr)
    print(f"{bar}\n", file=sys.stderr)
