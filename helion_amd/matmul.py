"""Drop-in for the reference's examples/matmul.py: ``matmul(x, y, epilogue)`` with the same signature, layouts and
output dtype (``promote_types(x.dtype, y.dtype)``), backed by the gfx950 HIP kernels.

The reference compiles whatever Python callable it is given into the kernel.  Here the epilogues its examples and
tests use — identity, ``acc + bias[tile[1]]`` and ``relu(acc + bias[tile[1]])`` — are fused into the HIP kernel when
they are passed as the :class:`BiasEpilogue` objects below (plain callables with the reference's ``(acc, tile)``
signature, so they also work with the reference's own kernel).  Any other callable is applied with torch to the fp32
accumulator the kernel returns: same result, one extra pass over the output."""
from __future__ import annotations

from typing import Callable

import torch
from torch import Tensor

from .ops import matmul_call


class BiasEpilogue:
    """``acc + bias[tile[1]]`` (examples/matmul.py:98), optionally followed by relu (:108-110).  ``bias``: ``[n]`` or
    ``[1, n]``."""

    def __init__(self, bias: Tensor | None, relu: bool = False) -> None:
        self.bias = bias
        self.relu = relu

    def __call__(self, acc: Tensor, tile: tuple) -> Tensor:
        if self.bias is not None:
            acc = acc + self.bias.reshape(-1)[tile[1]]
        return torch.relu(acc) if self.relu else acc


def bias_add(bias: Tensor) -> BiasEpilogue:
    return BiasEpilogue(bias, relu=False)


def bias_relu(bias: Tensor) -> BiasEpilogue:
    return BiasEpilogue(bias, relu=True)


def relu() -> BiasEpilogue:
    return BiasEpilogue(None, relu=True)


def _run(x: Tensor, y: Tensor, epilogue: Callable | None, split_k: int) -> Tensor:
    dt = torch.promote_types(x.dtype, y.dtype)
    if epilogue is None:
        return matmul_call(x, y, None, False, dt, split_k)
    if isinstance(epilogue, BiasEpilogue):
        return matmul_call(x, y, epilogue.bias, epilogue.relu, dt, split_k)
    # arbitrary callable: the kernel hands back the fp32 accumulator (examples/matmul.py:51-55: acc is fp32 and the
    # epilogue's result is cast on the store); the one-tile view of the reference's eager mode is tile = whole dims
    acc = matmul_call(x, y, None, False, torch.float32, split_k)
    m, n = acc.shape
    return epilogue(acc, (slice(0, m), slice(0, n))).to(dt)


def matmul(x: Tensor, y: Tensor, epilogue: Callable[[Tensor, tuple], Tensor] | None = None) -> Tensor:
    """``out = epilogue(fp32(x) @ fp32(y), (tile_m, tile_n)).to(promote_types(x.dtype, y.dtype))`` (reference:
    examples/matmul.py:25-56).  x: [m, k], y: [k, n]; row-major y is the fast layout.  ``epilogue=None`` is the
    reference's default ``lambda acc, tile: acc``.  When the output has too few tiles for the chip the library splits K
    on its own (deterministic fp32 partial sums; see matmul_split_k)."""
    return _run(x, y, epilogue, 0)


def matmul_tritonbench(a: Tensor, b: Tensor, bias: Tensor | None) -> Callable:
    """examples/matmul.py:124-139."""
    if bias is not None:
        return lambda: matmul(a, b, bias_add(bias))
    return lambda: matmul(a, b)


def check(m: int, k: int, n: int) -> None:
    """examples/matmul.py:75-120: plain, bias and bias+relu epilogues against torch (the last two once fused, once as
    the reference's own lambdas)."""
    from .testing import run_example

    x = torch.randn([m, k], device="cuda", dtype=torch.float16)
    y = torch.randn([k, n], device="cuda", dtype=torch.float16)
    bias = torch.randn([n], device="cuda", dtype=torch.float16)
    run_example(matmul, torch.matmul, (x, y))
    run_example(lambda x, y, bias: matmul(x, y, bias_add(bias)), lambda x, y, bias: torch.nn.functional.linear(x, y.T, bias),
                (x, y, bias))
    run_example(lambda x, y, bias: matmul(x, y, lambda acc, tile: acc + bias[tile[1]]),
                lambda x, y, bias: torch.nn.functional.linear(x, y.T, bias), (x, y, bias))
    run_example(lambda x, y: matmul(x, y, bias_relu(bias)), lambda x, y: torch.relu(x @ y + bias), (x, y))
    run_example(lambda x, y: matmul(x, y, lambda acc, tile: torch.relu(acc + bias[tile[1]])),
                lambda x, y: torch.relu(x @ y + bias), (x, y))


def main() -> None:
    """examples/matmul.py:143-148."""
    check(1024, 1024, 1024)


if __name__ == "__main__":
    main()
