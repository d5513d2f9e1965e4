"""Drop-in for the reference's examples/moe_matmul_ogs.py."""
from __future__ import annotations

import torch

from .ops import moe_matmul_ogs_call, moe_matmul_topk_call, moe_routing_call


def moe_matmul_ogs(A: torch.Tensor, W: torch.Tensor, expert_token_counts: torch.Tensor,
                   expert_token_offsets: torch.Tensor, sorted_to_orig_token_idx: torch.Tensor,
                   max_T_per_expert_tensor: torch.Tensor) -> torch.Tensor:
    """``C[r] = A[r] @ W[e]`` for every row r routed to expert e (reference: examples/moe_matmul_ogs.py:25-80).
    A: [T,K], W: [E,K,N]; returns [T,N] in promote_types(A.dtype, W.dtype).  As in the reference only the
    *numel* of ``max_T_per_expert_tensor`` is used."""
    return moe_matmul_ogs_call(A, W, expert_token_counts, expert_token_offsets, sorted_to_orig_token_idx,
                             int(max_T_per_expert_tensor.numel()))


def _routing_max_experts() -> int:
    """Experts the routing kernel's LDS tables hold: 512, or 2048 with the opt-in instantiation switched on."""
    from . import _lib
    return 2048 if _lib.load().hx_get_features() & _lib.HX_FEATURE_ROUTING_WIDE else 512


def moe_matmul_ogs_helion_kernel_args_gen(A: torch.Tensor, W: torch.Tensor, top1_expert_per_token: torch.Tensor):
    """examples/moe_matmul_ogs.py:84-121: stable sort of rows by expert, per-expert counts and offsets.
    On the GPU the three tables come from one routing kernel; the host synchronisation the reference has
    (``.item()`` for the size of the dummy tensor, :113) is kept because the signature needs that size."""
    E = W.size(0)
    device = A.device
    if A.is_cuda and E <= _routing_max_experts() and top1_expert_per_token.dtype in (torch.int32, torch.int64):
        counts, offsets, idx, max_count = moe_routing_call(top1_expert_per_token, E)
        return (A, W, counts, offsets, idx, torch.empty(int(max_count.item()), device=device))
    sorted_to_orig_token_idx = torch.argsort(top1_expert_per_token, stable=True).to(torch.int32)
    expert_token_counts = torch.bincount(top1_expert_per_token, minlength=E).to(torch.int32)
    expert_token_offsets = torch.empty(E + 1, dtype=torch.int32, device=device)
    expert_token_offsets[0] = 0
    expert_token_offsets[1:] = torch.cumsum(expert_token_counts, 0, dtype=torch.int32)
    max_T_per_expert = int(expert_token_counts.max().item())
    return (A, W, expert_token_counts, expert_token_offsets, sorted_to_orig_token_idx,
            torch.empty(max_T_per_expert, device=device))


def moe_matmul_topk(A: torch.Tensor, W: torch.Tensor, expert_ids: torch.Tensor, top_k: int = 1) -> torch.Tensor:
    """Top-k form without the replicated activations and without any host synchronisation: ``A`` is [T_tok, K],
    ``expert_ids`` holds T_tok*top_k ids (token-major, i.e. ``topk_indices.reshape(-1)``), the result is
    [T_tok*top_k, N] with row r = A[r // top_k] @ W[expert_ids[r]].  Equals
    ``moe_matmul_ogs(*moe_matmul_ogs_helion_kernel_args_gen(A.repeat_interleave(top_k, 0), W, expert_ids))``."""
    return moe_matmul_topk_call(A, W, expert_ids, int(top_k))


def moe_routing(expert_ids: torch.Tensor, num_experts: int):
    """(counts, offsets, sorted_to_orig_idx, max_count) as int32 device tensors from one kernel; the tensor form
    of examples/moe_matmul_ogs.py:98-113 with ``max_count`` left on the device."""
    return moe_routing_call(expert_ids, int(num_experts))


def moe_matmul_ogs_reference(A: torch.Tensor, W: torch.Tensor, top1_expert_per_token: torch.Tensor) -> torch.Tensor:
    """examples/moe_matmul_ogs.py:125-148 (pure torch; rows of unused experts are left as allocated)."""
    T, K = A.shape
    N = W.size(2)
    device, dtype = A.device, torch.promote_types(A.dtype, W.dtype)
    C = torch.empty(T, N, device=device, dtype=dtype)
    for e in range(W.size(0)):
        token_idx = (top1_expert_per_token == e).nonzero(as_tuple=True)[0]
        if token_idx.numel() == 0:
            continue
        C[token_idx] = A[token_idx] @ W[e]
    return C


def check(T: int, K: int, N: int, n_experts: int) -> None:
    """examples/moe_matmul_ogs.py:152-179: fp16 operands, random top-1 routing, kernel against the per-expert
    definition (rtol 1e-2, atol 1e-1 as in helion/_testing.py:341-349)."""
    from .testing import run_example

    dtype, device = torch.float16, "cuda"
    A = torch.randn(T, K, device=device, dtype=dtype)
    W = torch.randn(n_experts, K, N, device=device, dtype=dtype)
    top1_expert_per_token = torch.randint(n_experts, (T,), device=device)
    args = moe_matmul_ogs_helion_kernel_args_gen(A, W, top1_expert_per_token)
    run_example(lambda: moe_matmul_ogs(*args), lambda: moe_matmul_ogs_reference(A, W, top1_expert_per_token), ())


def main() -> None:
    """examples/moe_matmul_ogs.py:182-186."""
    check(1000, 500, 200, 30)


if __name__ == "__main__":
    main()
