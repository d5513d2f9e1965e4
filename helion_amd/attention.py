"""Drop-in for the reference's examples/attention.py: ``attention(q, k, v)`` with the same signature, layouts and output
dtype, backed by the gfx950 HIP kernels (16-bit MFMA flash attention for head_dim 64 / 128; a plain kernel for fp32
inputs and other shapes)."""
from __future__ import annotations

import math

import torch

from .ops import attention_call


def attention(q_in: torch.Tensor, k_in: torch.Tensor, v_in: torch.Tensor) -> torch.Tensor:
    """``softmax(q k^T / sqrt(head_dim)) v`` over the last two dimensions (reference: examples/attention.py:33-84).
    q: [..., seq_q, head_dim]; k, v: [..., seq_k, head_dim]; output: the shape and dtype of q.  As in the reference the
    softmax runs in base 2 with fp32 statistics and the probabilities are cast to the value dtype before the P.V
    product."""
    return attention_call(q_in, k_in, v_in)


# examples/attention.py:89-98: the reference re-registers the same body with dynamic shapes; one kernel serves both here
attention_dynamic = attention


def ref_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """The manual baseline of examples/attention.py:125-131."""
    p = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(q.size(-1))
    p = torch.softmax(p.float(), dim=-1).to(q.dtype)
    return torch.matmul(p, v)


def test(z: int, h: int, n_ctx: int, head_dim: int, dtype: torch.dtype = torch.float32,
         device: torch.device | str = "cuda") -> None:
    """examples/attention.py:104-145, against sdpa and the manual baseline (the reference's third baseline is a
    torch.compile'd flex_attention, which needs a compiler stack this package does not use)."""
    from .testing import run_example

    q, k, v = [torch.randn((z, h, n_ctx, head_dim), dtype=dtype, device=device) for _ in range(3)]
    baselines = {"torch": torch.nn.functional.scaled_dot_product_attention, "ref": ref_attention}
    run_example(attention, baselines, (q, k, v))


def main() -> None:
    """examples/attention.py:151-156."""
    test(2, 32, 1024, 64, torch.float16)


if __name__ == "__main__":
    main()
