"""GPU parity of hx_moe_grouped_gemm against the CPU oracle (= moe_matmul_ogs_reference semantics), the
golden fixture, ragged/empty-expert edge cases and sampled rows at the benchmark size."""
import pathlib

import numpy as np
import pytest
import torch

import helion_amd as hx
from helion_amd import inputs
from oracle import oracle as orc
from tests._util import TOL, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
G = pathlib.Path(__file__).resolve().parent / "golden"


def _run(A, W, ex):
    args = hx.moe_matmul_ogs_helion_kernel_args_gen(A.to(DEV), W.to(DEV), ex.to(DEV))
    return hx.moe_matmul_ogs(*args)


# path: what hx_moe_path reports - 0 the fp32-FMA kernel, 1 / 2 / 3 MFMA with 32- / 128- / 256-row tiles, 4 MFMA with
# 128-row tiles and a zero-filled partial last k-tile, 5 the same with A fetched in 4-byte pieces (K even, K % 8 != 0)
@pytest.mark.parametrize("T,K,N,E,topk,dtype,path", [
    (1000, 500, 200, 30, 1, torch.float16, 5),    # examples/moe_matmul_ogs.py:186: 8-byte rows, A by 4-byte DMA
    (1000, 504, 200, 30, 1, torch.float16, 4),    # ... the nearest shape with 16-byte rows: K = 7 k-tiles + 56
    (1000, 500, 200, 30, 1, torch.bfloat16, 5),
    (333, 2, 8, 3, 1, torch.bfloat16, 5),         # ... one pair of elements
    (700, 70, 136, 6, 2, torch.float16, 5),       # ... 64 + 6, top-2
    (40, 126, 64, 4, 1, torch.bfloat16, 5),       # ... 4-byte aligned rows only (K % 4 = 2), few rows
    (2500, 1030, 256, 2, 1, torch.bfloat16, 5),   # ... 16 tiles + 6, large experts
    (37, 101, 24, 3, 1, torch.bfloat16, 0),       # odd K: 2-byte aligned rows, the FMA kernel
    (512, 256, 512, 4, 1, torch.bfloat16, 2),
    (700, 128, 256, 5, 1, torch.float16, 2),
    (2048, 512, 768, 8, 2, torch.bfloat16, 2),    # top-2 expanded rows
    (8192, 192, 2048, 2, 1, torch.bfloat16, 3),   # 256-row tiles
    (300, 64, 256, 16, 1, torch.bfloat16, 2),     # most tiles nearly empty
    (37, 100, 19, 3, 1, torch.bfloat16, 0),       # N % 8 != 0: the FMA kernel
    (512, 128, 384, 4, 1, torch.bfloat16, 2),     # ragged last column tile (N % 128 = 0, N % 256 = 128)
    (600, 64, 1408, 8, 2, torch.float16, 2),      # N = 5.5 tiles of 256
    (256, 64, 8, 2, 1, torch.bfloat16, 2),        # a single column tile with one valid 16-byte chunk
    (300, 192, 200, 5, 1, torch.bfloat16, 2),     # N % 8 == 0, nothing else aligned
    (32, 256, 512, 8, 1, torch.bfloat16, 1),      # a decode batch: the 32-row tile kernel
    (16, 512, 264, 4, 2, torch.float16, 1),       # ... top-2, ragged last column tile
    (7, 64, 128, 3, 1, torch.bfloat16, 1),        # ... one k-tile, fewer rows than experts' tiles
    (24, 1024, 1408, 40, 1, torch.bfloat16, 1),   # ... more experts than rows
    (300, 8, 64, 3, 1, torch.bfloat16, 4),        # partial last k-tile: the only one, a single chunk
    (300, 72, 136, 3, 1, torch.float16, 4),       # ... one full tile + 8
    (1000, 120, 256, 7, 2, torch.bfloat16, 4),    # ... 64 + 56
    (20, 200, 264, 4, 1, torch.bfloat16, 4),      # ... few rows, 3 tiles + 8
    (5000, 1000, 512, 3, 1, torch.bfloat16, 4),   # ... large experts: 15 tiles + 40
    (6000, 64, 64, 700, 1, torch.bfloat16, 2),    # tile table built 256 experts at a time (three chunks, many empty)
    (9000, 128, 128, 300, 2, torch.float16, 2),   # ... two chunks, top-2
])
def test_shapes_vs_oracle(T, K, N, E, topk, dtype, path):
    A, W, ex = inputs.moe_inputs(T // topk, K, N, E, topk, seed=T + K, dtype=dtype)
    from helion_amd import _lib
    assert _lib.load().hx_moe_path(A.shape[0], K, N, E, 1, 1 << 20, 1 << 20, 1 << 20) == path
    out = _run(A, W, ex)
    assert out.dtype == dtype and out.shape == (A.shape[0], N)
    assert rel_err(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2


def test_golden_fixture():
    z = np.load(G / "moe_small.npz")
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        A = torch.from_numpy(z[f"{name}_A"].copy()).view(dt); W = torch.from_numpy(z[f"{name}_W"].copy()).view(dt)
        ex = torch.from_numpy(z[f"{name}_expert"].copy())
        ref = torch.from_numpy(z[f"{name}_out"].copy()).view(dt)
        assert rel_err(_run(A, W, ex), ref) <= 1e-2


@pytest.mark.parametrize("K,N", [(128, 256), (96, 40)])
def test_empty_experts_and_uncovered_rows_are_zero(K, N):
    A, W, ex = inputs.moe_inputs(400, K, N, 6, 1, seed=1, dtype=torch.bfloat16)
    ex[ex == 2] = 4  # expert 2 empty
    A_, W_, counts, offsets, idx, mt = hx.moe_matmul_ogs_helion_kernel_args_gen(A.to(DEV), W.to(DEV), ex.to(DEV))
    counts2 = counts.clone(); counts2[1] = 0  # expert 1 switched off: its rows must come out zero
    out = hx.moe_matmul_ogs(A_, W_, counts2, offsets, idx, mt).cpu()
    ref = orc.moe_matmul_ogs(A, W, counts2.cpu(), offsets.cpu(), idx.cpu())
    assert rel_err(out, ref) <= 1e-2
    assert bool((out[ex == 1] == 0).all())


def test_all_rows_one_expert_equals_dense_matmul():
    g = torch.Generator().manual_seed(2)
    A = torch.randn(512, 256, generator=g).bfloat16(); W = (torch.randn(3, 256, 256, generator=g) * 0.1).bfloat16()
    ex = torch.full((512,), 2)
    out = _run(A, W, ex)
    assert rel_err(out, (A.float() @ W[2].float()).bfloat16()) <= 1e-2


def test_c5_sampled_rows():
    A, W, ex = inputs.moe_c5()
    assert A.shape == (32768, 4096) and W.shape == (8, 4096, 14336)
    Ad, Wd, exd = A.to(DEV), W.to(DEV), ex.to(DEV)
    out = hx.moe_matmul_ogs(*hx.moe_matmul_ogs_helion_kernel_args_gen(Ad, Wd, exd))
    g = torch.Generator().manual_seed(0)
    for e in range(8):
        rows = (ex == e).nonzero(as_tuple=True)[0]
        pick = rows[torch.randperm(rows.numel(), generator=g)[:48]]
        ref = (A[pick].float() @ W[e].float()).bfloat16()
        assert rel_err(out[pick.to(DEV)], ref) <= 1e-2
    # top-2: the two rows of a token hold the same activations but different experts
    assert not torch.equal(out[0], out[1])


def test_random_shapes_vs_oracle():
    """A seeded sweep over row counts, K/N that land on the MFMA kernel (K % 64 == 0, N % 8 == 0, ragged last column
    tile included) and on the general kernel, expert counts, top-k and both 16-bit types; replicated and top-k entry."""
    rng = np.random.default_rng(7)
    for case in range(16):
        tokens = int(rng.choice([1, 50, 256, 700, 1500]))
        K = int(rng.choice([64, 128, 320, 100]))
        N = int(rng.choice([8, 256, 264, 384, 1000, 50]))
        E = int(rng.choice([1, 3, 8, 40]))
        topk = int(rng.choice([1, 2])) if E >= 2 else 1
        dtype = [torch.bfloat16, torch.float16][int(rng.integers(0, 2))]
        A, W, ex = inputs.moe_inputs(tokens, K, N, E, topk, seed=500 + case, dtype=dtype)
        ref = orc.moe_matmul_ogs_reference(A, W, ex)
        out = _run(A, W, ex)
        assert rel_err(out, ref) <= 1e-2, (case, tokens, K, N, E, topk, dtype)
        out2 = hx.moe_matmul_topk(A[::topk].contiguous().to(DEV), W.to(DEV), ex.to(DEV), topk)
        assert torch.equal(out, out2), (case, tokens, K, N, E, topk, dtype)
