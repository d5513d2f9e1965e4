"""GPU parity of the device-side routing kernel (hx_moe_routing) against the oracle's restatement of
examples/moe_matmul_ogs.py:98-113 (torch.argsort(stable=True) / bincount / cumsum): bit-exact integer tables; and of
the top-k entry point (hx_moe_topk_matmul) against the replicated-activation form the reference's caller builds."""
import pytest
import torch

import helion_amd as hx
from helion_amd import inputs
from oracle import oracle as orc
from tests._util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ids(T, E, seed, skew=1.2, dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -skew
    return torch.multinomial(p, T, replacement=True, generator=g).to(dtype) if T else torch.zeros(0, dtype=dtype)


def _check_tables(ids, E):
    counts, offsets, idx, max_count = hx.moe_routing(ids.to(DEV), E)
    _, _, rc, ro, ri, rmax = orc.moe_args_gen(torch.zeros(1, 1), torch.zeros(E, 1, 1), ids.long())
    assert counts.dtype == offsets.dtype == idx.dtype == max_count.dtype == torch.int32
    assert torch.equal(counts.cpu(), rc) and torch.equal(offsets.cpu(), ro)
    assert torch.equal(idx.cpu(), ri)
    assert int(max_count.item()) == rmax.numel()


@pytest.mark.parametrize("T,E", [(1, 1), (1, 8), (63, 8), (64, 8), (65, 3), (1000, 30), (1024, 512), (4097, 2), (16384, 8),
                                 (32768, 8), (50000, 257), (100003, 128), (1 << 20, 8), (300000, 512)])
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_routing_tables_bit_exact(T, E, dtype):
    _check_tables(_ids(T, E, seed=T + E, dtype=dtype), E)


def test_routing_degenerate_distributions():
    _check_tables(torch.full((5000,), 3), 7)                      # every row on one expert
    _check_tables(torch.arange(5000) % 11, 11)                    # round robin
    _check_tables(torch.arange(4999, -1, -1) % 64, 64)            # descending
    _check_tables(torch.zeros(0, dtype=torch.int64), 4)           # no rows
    _check_tables((torch.arange(3000) // 1000), 3)                # already sorted blocks


@pytest.mark.parametrize("T", [3000, 70001])   # one-workgroup and multi-workgroup forms
def test_routing_skips_out_of_range_ids(T):
    ids = _ids(T, 6, seed=9)
    ids[::7] = -1
    ids[3::11] = 6
    ids[5::13] = 1 << 40
    counts, offsets, idx, max_count = hx.moe_routing(ids.to(DEV), 6)
    ok = (ids >= 0) & (ids < 6)
    rows = torch.nonzero(ok).flatten()
    order = rows[torch.argsort(ids[rows], stable=True)]
    n = int(ok.sum())
    assert int(offsets[-1]) == n
    assert torch.equal(idx[:n].cpu().long(), order)
    assert bool((idx[n:] == -1).all())
    assert torch.equal(counts.cpu().long(), torch.bincount(ids[rows], minlength=6))


def test_routing_properties_at_benchmark_size():
    _, _, ex = inputs.moe_c5()
    counts, offsets, idx, max_count = (t.cpu().long() for t in hx.moe_routing(ex.to(DEV), 8))
    T = ex.numel()
    assert torch.equal(torch.sort(idx).values, torch.arange(T))      # a permutation
    se = ex[idx]
    assert bool((se[1:] >= se[:-1]).all())                           # grouped by expert
    same = se[1:] == se[:-1]
    assert bool((idx[1:][same] > idx[:-1][same]).all())              # ties keep the original order
    assert torch.equal(offsets[1:] - offsets[:-1], counts) and int(offsets[0]) == 0 and int(offsets[-1]) == T
    assert int(max_count) == int(counts.max())


@pytest.mark.parametrize("T_tok,K,N,E,topk,dtype", [
    (512, 256, 512, 4, 2, torch.bfloat16),     # tile256 kernel
    (300, 128, 256, 6, 4, torch.float16),
    (1000, 500, 200, 30, 1, torch.float16),    # the reference example's shape: A by 4-byte DMA
    (123, 96, 40, 5, 3, torch.bfloat16),
    (250, 500, 136, 7, 2, torch.bfloat16),     # ... with the top-k gather (row r reads A_tok[r / 2])
    (90, 120, 64, 6, 4, torch.float16),        # partial last k-tile with the top-k gather
    (64, 101, 24, 3, 2, torch.bfloat16),       # odd K: the FMA kernel
])
def test_topk_matmul_equals_replicated_form(T_tok, K, N, E, topk, dtype):
    A_rep, W, ex = inputs.moe_inputs(T_tok, K, N, E, topk, seed=T_tok + topk, dtype=dtype)
    A_tok = A_rep[::topk].contiguous()
    assert torch.equal(A_tok.repeat_interleave(topk, 0), A_rep)
    out = hx.moe_matmul_topk(A_tok.to(DEV), W.to(DEV), ex.to(DEV), topk)
    assert out.shape == (T_tok * topk, N) and out.dtype == dtype
    assert rel_err(out, orc.moe_matmul_ogs_reference(A_rep, W, ex)) <= 1e-2
    rep = hx.moe_matmul_ogs(*hx.moe_matmul_ogs_helion_kernel_args_gen(A_rep.to(DEV), W.to(DEV), ex.to(DEV)))
    assert torch.equal(out, rep)   # same kernel arithmetic, only the gather index differs


def test_topk_matmul_rows_with_invalid_ids_are_zero():
    A_rep, W, ex = inputs.moe_inputs(256, 128, 256, 4, 2, seed=5, dtype=torch.bfloat16)
    A_tok = A_rep[::2].contiguous()
    ex = ex.clone()
    ex[::5] = -1
    out = hx.moe_matmul_topk(A_tok.to(DEV), W.to(DEV), ex.to(DEV), 2).cpu()
    assert bool((out[ex == -1] == 0).all())
    keep = ex >= 0
    ref = orc.moe_matmul_ogs_reference(A_rep[keep], W, ex[keep])
    assert rel_err(out[keep], ref) <= 1e-2


def test_topk_matmul_c5_sampled_rows():
    A, W, ex = inputs.moe_c5()
    A_tok = A[::2].contiguous()
    out = hx.moe_matmul_topk(A_tok.to(DEV), W.to(DEV), ex.to(DEV), 2)
    g = torch.Generator().manual_seed(1)
    for e in range(8):
        rows = (ex == e).nonzero(as_tuple=True)[0]
        pick = rows[torch.randperm(rows.numel(), generator=g)[:32]]
        ref = (A[pick].float() @ W[e].float()).bfloat16()
        assert rel_err(out[pick.to(DEV)], ref) <= 1e-2
