"""The 16-bit siblings (dense matmul with fused epilogue and split-K, flash attention) and the casts / per-tensor
quantisation, executed on the CPU in the host execution model (tests/sim) against the oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests._util import rel_err
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn


def _mm(m, n, k, dt, col, bias, relu, split, od, path, splits=None, variant="lazy-reverse"):
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).to(dt)
    y = torch.randn(k, n, generator=g).to(dt)
    if col:
        y = y.t().contiguous().t()
    b = torch.randn(n, generator=g).to(dt) if bias else None
    simlib.configure(variant)
    out = simops.matmul(x, y, b, relu, od, split, want_path=path, want_splits=splits)
    ref = orc.matmul(x, y, b, relu, od or dt)
    assert rel_err(out, ref) <= 1e-2, (m, n, k, dt, col, bias, relu, split, od)


# path (hx_matmul_path): 1 = MFMA tile kernels, 0 = plain
@pytest.mark.parametrize("m,n,k,dt,col,bias,relu,split,od,path", [
    (256, 256, 128, torch.bfloat16, False, False, False, 1, None, 1),
    (300, 264, 192, torch.bfloat16, False, True, False, 1, None, 1),        # ragged rows and columns, bias
    (256, 256, 128, torch.float16, True, False, True, 1, None, 1),          # column-major second operand, relu
    (512, 256, 256, torch.bfloat16, False, True, True, 1, None, 1),
    (64, 64, 2048, torch.float16, False, False, False, 0, None, 1),         # the split-K example's shape class: library's choice
    (256, 512, 256, torch.bfloat16, False, True, False, 2, torch.float32, 1),  # forced two splits, raw fp32 accumulator out
    (128, 136, 320, torch.float16, False, True, True, 3, None, 1),
    (100, 50, 37, torch.float32, False, True, True, 1, None, 0),            # fp32 operands: plain kernel
    (33, 20, 64, torch.bfloat16, False, False, False, 1, None, 0),          # N % 8 != 0: plain kernel
])
def test_matmul(m, n, k, dt, col, bias, relu, split, od, path):
    _mm(m, n, k, dt, col, bias, relu, split, od, path)


def test_matmul_256_tile_kernel():
    # enough rows and columns that the library picks the 256x256 tile (the grouped GEMM's kernel with identity rows)
    _mm(2048, 2048, 128, torch.bfloat16, False, True, True, 1, None, 1)
    _mm(2048, 2304, 192, torch.float16, True, False, False, 1, None, 1, variant="lazy")


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
def test_matmul_every_variant(variant):
    _mm(384, 392, 256, torch.bfloat16, False, True, True, 2, None, 1, variant=variant)


@pytest.mark.parametrize("bh,m,n,d,dt,path", [
    (1, 128, 128, 128, torch.bfloat16, 1),
    (2, 200, 333, 64, torch.bfloat16, 1),     # ragged queries and keys
    (1, 64, 1000, 128, torch.float16, 1),
    (1, 300, 64, 64, torch.float16, 1),
    (3, 1, 77, 128, torch.bfloat16, 1),       # one query row
    (1, 33, 77, 32, torch.float32, 0),        # plain kernel
    (1, 40, 50, 96, torch.bfloat16, 0),
])
def test_attention16(bh, m, n, d, dt, path):
    g = torch.Generator().manual_seed(m + n)
    q = torch.randn(bh, m, d, generator=g).to(dt)
    k, v = (torch.randn(bh, n, d, generator=g).to(dt) for _ in range(2))
    ref = orc.attention(q, k, v)
    for variant in ("lazy-reverse", "eager-interleaved"):
        simlib.configure(variant)
        out = simops.attention16(q, k, v, want_path=path)
        assert rel_err(out, ref) <= 2e-2, variant


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
def test_attention16_every_variant(variant):
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 200, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    k, v = k.repeat(1, 3, 1)[:, :520], v.repeat(1, 3, 1)[:, :520]
    simlib.configure(variant)
    assert rel_err(simops.attention16(q, k.contiguous(), v.contiguous(), want_path=1), orc.attention(q, k, v)) <= 2e-2


def _same_codes(got, want, src):
    g, w = got.view(torch.uint8).reshape(-1), want.view(torch.uint8).reshape(-1)
    nan_src = torch.isnan(src.float()).reshape(-1)
    assert torch.equal(g[~nan_src], w[~nan_src])
    assert bool(((g[nan_src] & 0x7F) == 0x7F).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cast_every_16_bit_pattern(dtype):
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    simlib.configure("lazy")
    _same_codes(simops.cast_e4m3_x3(x, x, x)[1], x.to(E4), x)


@pytest.mark.parametrize("n", [1, 15, 16, 17, 4097])
def test_cast_ragged_lengths(n):
    g = torch.Generator().manual_seed(n)
    xs = [(torch.randn(n, generator=g) * 4).to(torch.float32) for _ in range(3)]
    simlib.configure("lazy")
    for o, x in zip(simops.cast_e4m3_x3(*xs), xs):
        _same_codes(o, x.to(E4), x)


@pytest.mark.parametrize("n,dtype", [(1, torch.float32), (1000, torch.bfloat16), (70000, torch.float16), (4096, torch.float32)])
def test_quantize_per_tensor(n, dtype):
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(n, generator=g) * 3).to(dtype)
    simlib.configure("lazy")
    q, scale = simops.fp8_quantize(x)
    rq, rs = orc.fp8_quantize_per_tensor(x)
    assert float(scale) == float(rs)
    assert torch.equal(q.view(torch.uint8), rq.view(torch.uint8))


# ---- opt-in: the dense 256x256 kernel in persistent workgroups (HX_FEATURE_MATMUL_PERSISTENT, hx_matmul_path 2) -------------
@pytest.mark.parametrize("m,n,k,cus,variant,dtype", [(3072, 3072, 256, 8, "lazy", torch.bfloat16),
                                                     (2304, 4096, 384, 16, "eager-interleaved", torch.float16)])
def test_persistent_dense_matmul(m, n, k, cus, variant, dtype):
    """144 tiles on 8 / 16 persistent workgroups: every tile's epilogue runs inside the next tile's first k-tile.  Bit-equal
    to the kernel it replaces (same MFMA order per accumulator)."""
    from helion_amd import _lib
    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn(m, k, generator=g) * 0.5).to(dtype)
    y = (torch.randn(k, n, generator=g) * 0.5).to(dtype)
    simlib.configure(variant)
    with simlib.cus(cus):
        base = simops.matmul(x, y, want_path=1)
        with simlib.features(_lib.HX_FEATURE_MATMUL_PERSISTENT):
            simlib.work()
            out = simops.matmul(x, y, want_path=2)
            w = simlib.work()
            assert simlib.load().hx_matmul_path(m, n + 8, k, k, n + 8, 1, n + 8, _lib.HX_BF16, None, None, None, None) == 1  # ragged column tile
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    assert rel_err(out, orc.matmul(x, y)) <= 1e-2
    assert w["workgroups"] == cus and w["mfma"] == (m // 256) * (n // 256) * (k // 64) * 512
