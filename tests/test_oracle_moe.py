"""Pins oracle.moe_* : routing-table invariants (library routines + definitions), the per-expert dense
definition (examples/moe_matmul_ogs.py:125-148) and an independent float64 brute force in C.
The reference's own unit test skips accuracy for this kernel (test/test_examples.py:434-458)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc


def _case(T, K, N, E, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    A = torch.randn(T, K, generator=g).to(dtype)
    W = torch.randn(E, K, N, generator=g).to(dtype)
    ex = torch.randint(E, (T,), generator=g)
    return A, W, ex


def test_args_gen_invariants():
    A, W, ex = _case(200, 8, 8, 7, 0, torch.float16)
    ex[ex == 3] = 2  # make expert 3 empty
    _, _, counts, offsets, idx, max_t = orc.moe_args_gen(A, W, ex)
    assert counts.dtype == offsets.dtype == idx.dtype == torch.int32
    assert int(offsets[0]) == 0 and int(offsets[-1]) == 200
    assert torch.equal(offsets[1:] - offsets[:-1], counts)
    assert int(counts[3]) == 0
    assert torch.equal(torch.sort(idx.long()).values, torch.arange(200))  # a permutation
    sorted_e = ex[idx.long()]
    assert bool((sorted_e[1:] >= sorted_e[:-1]).all())
    for e in range(7):  # stable: original order kept inside an expert
        seg = idx[int(offsets[e]) : int(offsets[e + 1])].long()
        assert bool((seg[1:] > seg[:-1]).all())
        assert bool((ex[seg] == e).all())
    assert max_t.numel() == int(counts.max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kernel_semantics_equal_reference_definition(dtype):
    A, W, ex = _case(150, 24, 20, 6, 1, dtype)
    args = orc.moe_args_gen(A, W, ex)
    assert torch.equal(orc.moe_matmul_ogs(*args), orc.moe_matmul_ogs_reference(A, W, ex))


@pytest.mark.parametrize("dtype,is_bf16", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_against_float64_bruteforce(oracle_c, dtype, is_bf16):
    T, K, N, E = 40, 17, 9, 4
    A, W, ex = _case(T, K, N, E, 2, dtype)
    out = np.empty((T, N), dtype=np.float64)
    ab = A.view(torch.int16).numpy().copy(); wb = W.view(torch.int16).numpy().copy()
    eb = ex.to(torch.int32).numpy().copy()
    oracle_c.orc_moe_f64(ab.ctypes.data, wb.ctypes.data, eb.ctypes.data, out.ctypes.data, T, K, N, is_bf16)
    got = orc.moe_matmul_ogs(*orc.moe_args_gen(A, W, ex)).double().numpy()
    ulp = 2.0**-7 if is_bf16 else 2.0**-10
    assert np.all(np.abs(got - out) <= ulp * np.maximum(np.abs(out), 1e-3))


def test_uncovered_rows_are_zero_and_partial_tables_respected():
    A, W, ex = _case(30, 8, 8, 3, 3, torch.float16)
    _, _, counts, offsets, idx, mt = orc.moe_args_gen(A, W, ex)
    counts2 = counts.clone(); counts2[1] = 0  # drop expert 1 without touching offsets
    out = orc.moe_matmul_ogs(A, W, counts2, offsets, idx, mt)
    rows1 = (ex == 1).nonzero(as_tuple=True)[0]
    assert bool((out[rows1] == 0).all())
    full = orc.moe_matmul_ogs(A, W, counts, offsets, idx, mt)
    rest = (ex != 1).nonzero(as_tuple=True)[0]
    assert torch.equal(out[rest], full[rest])


def test_single_expert_is_a_plain_matmul():
    A, W, _ = _case(12, 16, 8, 1, 4, torch.bfloat16)
    ex = torch.zeros(12, dtype=torch.long)
    out = orc.moe_matmul_ogs(*orc.moe_args_gen(A, W, ex))
    assert torch.equal(out, (A.float() @ W[0].float()).to(torch.bfloat16))
