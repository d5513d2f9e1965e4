"""The reference's own checks for the path - every `check(...)` call of the example scripts' `main()` and the shapes of
its test_examples.py for these kernels - executed in the host execution model (tests/sim) against the oracle, with the
inputs built the way the scripts build them (same dtypes, same layouts: a row-major `y`, `v` given as [B, H, S, D] and
permuted by strides, routing tables made from random expert ids).  The GPU twin is tests/test_gpu_example_scripts.py.

    examples/fp8_gemm.py:117-119           check(256, 256, 256), (512, 512, 512), (1024, 1024, 1024)
    examples/fp8_attention.py:292-294      check(1, 2, 128, 64), (2, 4, 256, 64), (4, 8, 512, 128)
    examples/moe_matmul_ogs.py:186         check(1000, 500, 200, 30)
    examples/matmul.py:147                 check(1024, 1024, 1024)            (plain, + bias epilogue)
    examples/matmul_split_k.py:123         check(64, 32768, 64)
    examples/attention.py:151-156          batch 2, 32 heads, 1024 x 64, float16 (here: 4 of the 64 heads; all under HX_SIM_SWEEP=1)
    test/test_examples.py:117              fp8_gemm 256 x 256;  :577 fp8_attention (2, 4, 256, 64);  :435 moe (1000, 500, 200, 30);
                                           :460 matmul_split_k (64, 1024, 64);  :342-392 attention (1, 32, 512, 64)
"""
import os

import pytest
import torch

from oracle import oracle as orc
from tests._util import attention_close, rel_err
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn
SWEEP = os.environ.get("HX_SIM_SWEEP") == "1"


@pytest.mark.parametrize("m,k,n", [(256, 256, 256), (512, 512, 512), (1024, 1024, 1024)])
def test_fp8_gemm_check(m, k, n):
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, k, generator=g).to(E4)
    y = torch.randn(k, n, generator=g).to(E4)   # row-major, as the script makes it
    simlib.configure("lazy")
    out = simops.fp8_gemm(x, y, None, None, torch.float16, want_path=4)
    ref = orc.fp8_gemm_ref_eager(x, y, torch.float16)
    assert rel_err(out, ref) <= 1e-2
    torch.testing.assert_close(out.float(), ref.float(), atol=1e-2 * float(ref.float().abs().max()), rtol=1e-2)


@pytest.mark.parametrize("batch,heads,seq,dim", [(1, 2, 128, 64), (2, 4, 256, 64), (4, 8, 512, 128)])
def test_fp8_attention_check(batch, heads, seq, dim):
    torch.manual_seed(42)  # (the script's seed)
    q, k, v = (torch.randn(batch, heads, seq, dim, dtype=torch.float16) for _ in range(3))
    simlib.configure("lazy-reverse")
    q8, k8, v8 = simops.cast_e4m3_x3(q, k, v)                     # the cast kernel; v stays [B, H, S, D]
    rq, rk, rv = orc.preprocess_fp8_attention_inputs(q, k, v)     # v permuted to [BH, D, S]
    assert torch.equal(q8.view(torch.uint8).reshape(rq.shape), rq.view(torch.uint8))
    assert torch.equal(v8.view(torch.uint8).reshape(batch * heads, seq, dim).transpose(1, 2), rv.view(torch.uint8))
    bh = batch * heads
    # the op hands the kernel v's memory as it is ([S][D] per head) with the strides of the permuted view
    out = simops.fp8_attention(q8.reshape(bh, seq, dim), k8.reshape(bh, seq, dim), rv, batch, heads, E4, True, "SD", want_path=1)
    ref = orc.fp8_attention(rq, rk, rv, batch, heads, E4)
    assert attention_close(out.float(), ref.float())
    torch.testing.assert_close(out.float(), ref.float(), atol=0.1, rtol=0.1)  # the script's own tolerance


def test_moe_matmul_ogs_check():
    T, K, N, E = 1000, 500, 200, 30
    g = torch.Generator().manual_seed(0)
    A = torch.randn(T, K, generator=g).to(torch.float16)
    W = torch.randn(E, K, N, generator=g).to(torch.float16)
    ex = torch.randint(E, (T,), generator=g)
    simlib.configure("lazy")
    counts, offsets, idx, mx = simops.moe_routing(ex, E)          # the routing-table kernel in place of the script's torch ops
    _, _, rc, ro, ri, _ = orc.moe_args_gen(A, W, ex)
    assert torch.equal(counts, rc) and torch.equal(offsets, ro) and torch.equal(idx, ri) and int(mx) == int(rc.max())
    out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=5, poison=5.0)
    ref = orc.moe_matmul_ogs_reference(A, W, ex)
    torch.testing.assert_close(out.float(), ref.float(), atol=1e-2 * float(ref.float().abs().max()), rtol=1e-2)


def test_matmul_check_plain_and_bias():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1024, 1024, generator=g).to(torch.float16)
    y = torch.randn(1024, 1024, generator=g).to(torch.float16)
    bias = torch.randn(1024, generator=g).to(torch.float16)
    simlib.configure("lazy")
    out = simops.matmul(x, y)
    assert rel_err(out, orc.matmul(x, y)) <= 1e-2
    out = simops.matmul(x, y, bias=bias)
    assert rel_err(out, orc.matmul(x, y, bias)) <= 1e-2


@pytest.mark.parametrize("m,k,n", [(64, 32768, 64), (64, 1024, 64)])
def test_matmul_split_k_check(m, k, n):
    g = torch.Generator().manual_seed(k)
    x = torch.randn(m, k, generator=g).to(torch.float16)
    y = torch.randn(k, n, generator=g).to(torch.float16)
    bias = torch.randn(n, generator=g).to(torch.float16)
    simlib.configure("lazy-reverse")
    out = simops.matmul(x, y, split_k=0)   # 0: the library picks the split, as matmul_split_k does
    assert rel_err(out, orc.matmul(x, y)) <= 1e-2
    out = simops.matmul(x, y, bias=bias, split_k=0)
    assert rel_err(out, orc.matmul(x, y, bias)) <= 1e-2


@pytest.mark.parametrize("batch,heads,seq,dim,dtype", [(2, 32, 1024, 64, torch.float16), (1, 32, 512, 64, torch.bfloat16)])
def test_attention_check(batch, heads, seq, dim, dtype):
    g = torch.Generator().manual_seed(seq)
    bh = batch * heads if SWEEP else 4
    q, k, v = (torch.randn(bh, seq, dim, generator=g).to(dtype) for _ in range(3))
    simlib.configure("lazy")
    out = simops.attention16(q, k, v)
    ref = orc.attention(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0))[0]
    torch.testing.assert_close(out.float(), ref.float(), atol=1e-2, rtol=1e-2)


def test_the_smoke_run_case_by_case():
    """The cases of `__graft_entry__.smoke()` (same seeded inputs, same tolerances) in the host execution model, so that a
    change that would break the smoke run on the GPU is seen on the CPU first."""
    from helion_amd import inputs

    def rel(a, b):
        return float((a.float() - b.float()).abs().max() / b.float().abs().max())

    simlib.configure("lazy")
    a, b, sa, sb = inputs.gemm_scaled(256, 512, 384, 1)
    assert rel(simops.fp8_gemm(a, b, sa, sb, torch.bfloat16), orc.fp8_gemm(a, b, sa, sb, torch.bfloat16)) <= 1e-2
    a, b, sa, sb = inputs.gemm_scaled(16, 256, 1024, 2)
    assert rel(simops.fp8_gemm(a, b, sa, sb, torch.bfloat16, want_path=2), orc.fp8_gemm(a, b, sa, sb, torch.bfloat16)) <= 1e-2
    for s, seed in ((256, 3), (208, 4)):   # 208: a partial last key tile
        q, k, v = inputs.attention_inputs(1, 2, s, 128, seed)
        out = simops.fp8_attention(q, k, v, 1, 2, torch.float32, True, "DS", want_path=1)
        assert rel(out, orc.fp8_attention(q, k, v, 1, 2, torch.float32)) <= 2e-2
    for (T, K, N, E, seed), path in (((300, 120, 256, 5, 6), 4), ((512, 256, 512, 4, 4), 2)):   # K = 120: a partial last k-tile
        A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed)
        counts, offsets, idx, _ = simops.moe_routing(ex, E)
        out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=path, poison=2.0)
        assert rel(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2
    g = torch.Generator().manual_seed(5)
    x = torch.randn(300, 256, generator=g).bfloat16()
    y = torch.randn(256, 264, generator=g).bfloat16()
    bias = torch.randn(264, generator=g).bfloat16()
    assert rel(simops.matmul(x, y, bias=bias, relu=True), orc.matmul(x, y, bias, relu=True)) <= 1e-2
    q, k, v = (torch.randn(2, 2, 192, 128, generator=g).half() for _ in range(3))
    out = simops.attention16(q.reshape(4, 192, 128), k.reshape(4, 192, 128), v.reshape(4, 192, 128))
    assert rel(out, orc.attention(q, k, v).reshape(4, 192, 128)) <= 2e-2
