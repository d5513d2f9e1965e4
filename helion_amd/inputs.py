"""Seeded synthetic inputs for the benchmark / parity configurations.  All randomness comes from a CPU
``torch.Generator`` so the same seed gives the same bytes on any box; tensors are built on the CPU and
moved to ``device`` by the caller-facing helpers."""
from __future__ import annotations

import torch

E4M3 = torch.float8_e4m3fn


def _colmajor(t: torch.Tensor) -> torch.Tensor:
    """[K,N] tensor with strides (1,K)."""
    return t.T.contiguous().T


def gemm_c1(device="cpu"):
    """A[1024,1024] @ B[1024,1024], N(0,1) clamped to +-448, B column-major, unit scales."""
    g = torch.Generator().manual_seed(0)
    a = torch.randn(1024, 1024, generator=g).clamp(-448, 448).to(E4M3)
    b = _colmajor(torch.randn(1024, 1024, generator=g).clamp(-448, 448).to(E4M3))
    return a.to(device), b.to(device)


def gemm_scaled(m: int, n: int, k: int, seed: int, device="cpu"):
    """N(0,1)*0.5 e4m3 operands, B column-major, per-tensor fp32 scales uniform in [0.5,2]."""
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4M3)
    b = (torch.randn(n, k, generator=g) * 0.5).to(E4M3).T  # [k,n] view with strides (1,k)
    sa = torch.rand((), generator=g) * 1.5 + 0.5
    sb = torch.rand((), generator=g) * 1.5 + 0.5
    return a.to(device), b.to(device), sa.to(device), sb.to(device)


def gemm_c2(device="cpu"):
    return gemm_scaled(8192, 8192, 8192, 1, device)


def gemm_c3(device="cpu"):
    return gemm_scaled(16, 28672, 8192, 2, device)


def attention_inputs(batch: int, heads: int, seq: int, dim: int, seed: int, device="cpu"):
    """q,k,v ~ N(0,1) fp32 [B,H,S,D] -> e4m3 q,k [BH,S,D] and v [BH,D,S] (permute before the cast)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, heads, seq, dim, generator=g)
    k = torch.randn(batch, heads, seq, dim, generator=g)
    v = torch.randn(batch, heads, seq, dim, generator=g)
    q8 = q.to(E4M3).reshape(batch * heads, seq, dim)
    k8 = k.to(E4M3).reshape(batch * heads, seq, dim)
    v8 = v.permute(0, 1, 3, 2).to(E4M3).reshape(batch * heads, dim, seq).contiguous()
    return q8.to(device), k8.to(device), v8.to(device)


def attention_c4(device="cpu"):
    return attention_inputs(4, 32, 4096, 128, 3, device)


def moe_inputs(tokens: int, k: int, n: int, experts: int, topk: int, seed: int, dtype=torch.bfloat16, device="cpu",
               zipf_s: float = 1.2):
    """Zipf(s)-skewed top-k routing without replacement; rows are (token, slot) pairs, A is pre-expanded.
    Returns (A [tokens*topk, k], W [experts, k, n], expert_rows [tokens*topk] int64)."""
    g = torch.Generator().manual_seed(seed)
    p = torch.arange(1, experts + 1, dtype=torch.float32) ** (-zipf_s)
    sel = torch.multinomial(p.expand(tokens, experts), topk, replacement=False, generator=g)
    expert_rows = sel.reshape(-1)
    a_tok = torch.randn(tokens, k, generator=g).to(dtype)
    a = a_tok.repeat_interleave(topk, 0)
    w = torch.empty(experts, k, n, dtype=dtype)
    for e in range(experts):  # per-expert to bound the fp32 temporary
        w[e] = (torch.randn(k, n, generator=g) * 0.02).to(dtype)
    return a.to(device), w.to(device), expert_rows.to(device)


def moe_c5(device="cpu"):
    return moe_inputs(16384, 4096, 14336, 8, 2, 4, torch.bfloat16, device)
