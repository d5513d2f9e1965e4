"""Drop-in for the reference's examples/matmul_split_k.py: ``matmul_split_k(x, y, epilogue)``, a matmul that spreads
the K dimension over workgroups when the output alone has too few tiles to fill the chip (64 x 32768 x 64 is the
example's case).  The reference accumulates the splits with atomics in the output dtype and applies the epilogue to
the first split only; here the splits are fp32 partial sums added in a fixed order and the epilogue sees the whole
sum, which is what the reference computes with one split (its eager mode)."""
from __future__ import annotations

from typing import Callable

import torch
from torch import Tensor

from .matmul import _run, bias_add


def matmul_split_k(x: Tensor, y: Tensor, epilogue: Callable[[Tensor, tuple], Tensor] | None = None, *,
                   split_k: int = 0) -> Tensor:
    """examples/matmul_split_k.py:30-68.  ``split_k`` (keyword-only extension; the reference's is an autotuned
    parameter): 0 lets the library choose, n forces n splits."""
    return _run(x, y, epilogue, split_k)


def matmul_split_k_tritonbench(a: Tensor, b: Tensor, bias: Tensor | None) -> Callable:
    """examples/matmul_split_k.py:99-116."""
    if bias is not None:
        return lambda: matmul_split_k(a, b, bias_add(bias))
    return lambda: matmul_split_k(a, b)


def check(m: int, k: int, n: int) -> None:
    """examples/matmul_split_k.py:72-95."""
    from .testing import run_example

    x = torch.randn([m, k], device="cuda", dtype=torch.float16)
    y = torch.randn([k, n], device="cuda", dtype=torch.float16)
    run_example(lambda x, y: matmul_split_k(x, y), lambda x, y: torch.matmul(x, y), (x, y), atol=1)
    bias = torch.randn([n], device="cuda", dtype=torch.float16)
    run_example(lambda x, y: matmul_split_k(x, y, epilogue=lambda acc, tile: acc + bias[tile[1]]),
                lambda x, y: torch.nn.functional.linear(x, y.T, bias), (x, y), atol=1)
    run_example(lambda x, y: matmul_split_k(x, y, epilogue=bias_add(bias)),
                lambda x, y: torch.nn.functional.linear(x, y.T, bias), (x, y), atol=1)


def main() -> None:
    """examples/matmul_split_k.py:120-124."""
    check(64, 32768, 64)


if __name__ == "__main__":
    main()
