"""Drop-in for the reference's examples/fp8_attention.py."""
from __future__ import annotations

import math
from typing import Callable

import torch

from .ops import cast_e4m3_x3_call, fp8_attention_call


def fp8_attention_kernel(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, batch: int, heads: int, *,
                         out_dtype: torch.dtype = torch.float8_e4m3fn, exact_max: bool = True) -> torch.Tensor:
    """Scaled dot-product attention on e4m3 tensors (reference: examples/fp8_attention.py:22-106).
    q, k: [batch*heads, seq, dim]; v: [batch*heads, dim, seq] (pre-transposed); returns
    [batch, heads, seq, dim] float8_e4m3fn.  ``exact_max=True`` (default) quantises the un-normalised
    probabilities against the exact row max, which is what the reference computes when its kernel body
    is executed with one tile per loop; ``exact_max=False`` is the single-pass online softmax."""
    return fp8_attention_call(q, k, v, batch, heads, out_dtype, int(exact_max))


def preprocess_fp8_attention_inputs(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
    """examples/fp8_attention.py:110-133: cast to e4m3 (v permuted to [B,H,D,S] first), flatten batch*heads.
    The permute-then-cast of the reference keeps v's memory in [B,H,S,D] order (only the strides change), so on the
    GPU all three tensors go through one cast kernel and v comes back as the same strided view."""
    batch, heads, seq_len, head_dim = q.shape
    if (q.is_cuda and q.dtype == k.dtype == v.dtype and q.dtype in (torch.float16, torch.bfloat16, torch.float32)
            and q.shape == k.shape == v.shape and q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
        q_fp8, k_fp8, v_fp8 = cast_e4m3_x3_call(q, k, v)
        return (q_fp8.reshape(batch * heads, seq_len, head_dim), k_fp8.reshape(batch * heads, seq_len, head_dim),
                v_fp8.permute(0, 1, 3, 2).reshape(batch * heads, head_dim, seq_len))
    q_fp8 = q.to(torch.float8_e4m3fn)
    k_fp8 = k.to(torch.float8_e4m3fn)
    v = v.permute(0, 1, 3, 2)
    v_fp8 = v.to(torch.float8_e4m3fn)
    batch, heads, seq_len, head_dim = q.shape
    return (q_fp8.reshape(batch * heads, seq_len, head_dim), k_fp8.reshape(batch * heads, seq_len, head_dim),
            v_fp8.reshape(batch * heads, head_dim, seq_len))


def fp8_attention_tritonbench(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> Callable[[], torch.Tensor]:
    """examples/fp8_attention.py:137-154: preprocessing hoisted out of the returned thunk."""
    batch, heads, seq_len, head_dim = q.shape
    q_fp8, k_fp8, v_fp8 = preprocess_fp8_attention_inputs(q, k, v)
    return lambda: fp8_attention_kernel(q_fp8, k_fp8, v_fp8, batch, heads)


def _fp8_attention_pytorch_impl(q_fp8: torch.Tensor, k_fp8: torch.Tensor, v_fp8: torch.Tensor, batch: int, heads: int,
                                seq_len: int, head_dim: int) -> torch.Tensor:
    """The reference's torch baseline (examples/fp8_attention.py:158-238), head by head with torch._scaled_mm.  Its
    numerics differ from the kernel's on purpose: it normalises p by its row sum *before* the e4m3 cast."""
    log2e = 1.44269504
    sm_scale = 1.0 / math.sqrt(float(head_dim))
    one = torch.tensor(1.0, device=q_fp8.device)
    heads_out = []
    for i in range(batch * heads):
        k_t = k_fp8[i].contiguous().t()                       # [dim, seq], column-major as _scaled_mm wants
        qk = torch._scaled_mm(q_fp8[i], k_t, one, one, use_fast_accum=False, out_dtype=torch.float32)
        qk_max = torch.amax(qk, dim=-1, keepdim=True)
        p = torch.exp2((qk * sm_scale - qk_max * sm_scale) * log2e)
        p8 = (p / p.sum(dim=-1, keepdim=True)).to(torch.float8_e4m3fn)
        v_t = v_fp8[i].contiguous().t()                       # [seq, dim], column-major
        o = torch._scaled_mm(p8, v_t, one, one, use_fast_accum=False, out_dtype=torch.float32)
        heads_out.append(o.to(torch.float8_e4m3fn))
    return torch.stack(heads_out, dim=0).reshape(batch, heads, seq_len, head_dim)


def fp8_attention_pytorch(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> Callable[[], torch.Tensor]:
    """examples/fp8_attention.py:242-256: the baseline as a thunk, preprocessing hoisted out of it."""
    batch, heads, seq_len, head_dim = q.shape
    q_fp8, k_fp8, v_fp8 = preprocess_fp8_attention_inputs(q, k, v)
    return lambda: _fp8_attention_pytorch_impl(q_fp8, k_fp8, v_fp8, batch, heads, seq_len, head_dim)


def check(batch: int, heads: int, seq_len: int, head_dim: int) -> None:
    """examples/fp8_attention.py:260-283: kernel against the torch baseline, atol = rtol = 0.1, then a timing table."""
    from .testing import run_example

    torch.manual_seed(42)
    q, k, v = (torch.randn(batch, heads, seq_len, head_dim, dtype=torch.float16, device="cuda") for _ in range(3))
    run_example(fp8_attention_tritonbench(q, k, v), fp8_attention_pytorch(q, k, v), (), atol=0.1, rtol=0.1)


def main() -> None:
    """examples/fp8_attention.py:287-295."""
    check(1, 2, 128, 64)
    check(2, 4, 256, 64)
    check(4, 8, 512, 128)


if __name__ == "__main__":
    main()
