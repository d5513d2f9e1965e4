"""GPU parity of hx_matmul (the 16-bit siblings of the fp8 GEMM: examples/matmul.py, examples/matmul_split_k.py of the
reference) against the CPU oracle, through the C ABI via the registered op.  Bar: max|out - ref| <= 2e-2 max|ref|
after rounding to the output type (the 16-bit kernels differ from the oracle only in fp32 summation order)."""
import pathlib

import numpy as np
import pytest
import torch

import helion_amd as hx
from helion_amd import _lib
from helion_amd.matmul import bias_add, bias_relu, relu
from oracle import oracle as orc
from tests._util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
_DT = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def _mk(m, k, n, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(m, k, generator=g).to(dtype), torch.randn(k, n, generator=g).to(dtype),
            torch.randn(n, generator=g).to(dtype))


def _path(x, y):
    m, k = x.shape; n = y.shape[1]
    return _lib.load().hx_matmul_path(m, n, k, x.stride(0), y.stride(0), y.stride(1), n, _DT[x.dtype], x.data_ptr(),
                                      y.data_ptr(), x.data_ptr(), None)


@pytest.mark.parametrize("m,k,n,path", [
    (256, 256, 256, 1), (1024, 1024, 1024, 1), (512, 64, 768, 1), (300, 192, 200, 1), (1, 64, 8, 1), (1000, 512, 1016, 1),
    (128, 128, 128, 1), (4096, 128, 2048, 1), (3000, 64, 4000, 1),   # the last two: enough tiles for the 256x256 kernel
    (64, 100, 64, 0), (33, 64, 7, 0), (5, 3, 2, 0),
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_shapes_and_epilogues_vs_oracle(m, k, n, path, dtype):
    x, y, bias = _mk(m, k, n, dtype, m + 3 * k + 7 * n)
    xd, yd, bd = x.to(DEV), y.to(DEV), bias.to(DEV)
    assert _path(xd, yd) == path
    for ep, kw in ((None, {}), (bias_add(bd), dict(bias=bias)), (bias_relu(bd), dict(bias=bias, relu=True)), (relu(), dict(relu=True))):
        out = hx.matmul(xd, yd, ep)
        assert out.dtype == dtype and out.shape == (m, n)
        assert rel_err(out, orc.matmul(x, y, **kw)) <= 1e-2


@pytest.mark.parametrize("m,k,n", [(256, 256, 256), (300, 192, 200), (1000, 512, 1016), (64, 4096, 72), (1, 64, 8), (4096, 128, 2056)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_column_major_y_in_place(m, k, n, dtype):
    """y given as the transpose of an [n, k] weight (what `x @ w.T` of a linear layer passes): read in place by the tile
    kernel, bit-identical to the row-major result (same MFMA operands in the same order)."""
    x, y, bias = _mk(m, k, n, dtype, m + k + n)
    xd, bd = x.to(DEV), bias.to(DEV)
    w = y.t().contiguous().to(DEV)            # [n, k]
    yc = w.t()                                # [k, n] with strides (1, k)
    assert _path(xd, yc) == 1
    for ep, kw in ((None, {}), (bias_relu(bd), dict(bias=bias, relu=True))):
        out = hx.matmul(xd, yc, ep)
        assert rel_err(out, orc.matmul(x, y, **kw)) <= 1e-2
        assert torch.equal(out, hx.matmul(xd, y.to(DEV), ep))
    assert torch.equal(hx.matmul_split_k(xd, yc, split_k=2), hx.matmul_split_k(xd, y.to(DEV), split_k=2))


def test_callable_epilogues_match_fused_ones():
    """The reference's own lambdas (examples/matmul.py:98,108-110; test/test_examples.py:143-200, bias of shape [1, n]
    indexed by the whole tile tuple) give what the fused epilogue objects give."""
    x, y, bias = _mk(512, 256, 384, torch.float16, 5)
    xd, yd, bd = x.to(DEV), y.to(DEV), bias.to(DEV)
    a = hx.matmul(xd, yd, lambda acc, tile: acc + bd[tile[1]])
    assert torch.equal(a, hx.matmul(xd, yd, bias_add(bd)))
    b2 = bd.reshape(1, -1)
    r = hx.matmul(xd, yd, lambda acc, tile: torch.relu(acc + b2[tile]))
    assert torch.equal(r, hx.matmul(xd, yd, bias_relu(bd)))
    assert rel_err(r, orc.matmul(x, y, bias, relu=True)) <= 1e-2
    r2 = hx.matmul(xd, yd, lambda acc, _: torch.nn.functional.relu(acc))
    assert torch.equal(r2, hx.matmul(xd, yd, relu()))


def test_fp32_operands_and_mixed_dtypes():
    """test/test_examples.py:33-46 feeds fp32 matrices: they run the plain fp32 kernel."""
    x, y, bias = _mk(128, 128, 128, torch.float32, 9)
    out = hx.matmul(x.to(DEV), y.to(DEV))
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), orc.matmul(x, y), atol=1e-4, rtol=1e-5)
    out = hx.matmul(x.to(DEV).half(), y.to(DEV), bias_add(bias.to(DEV)))     # promote_types(fp16, fp32) = fp32
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), orc.matmul(x.half(), y, bias), atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("m,k,n", [(64, 32768, 64), (64, 1024, 64), (256, 4096, 512), (100, 8192, 72)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_k_vs_oracle(m, k, n, dtype):
    """examples/matmul_split_k.py:120-124 (64 x 32768 x 64) and test/test_examples.py:460-474 (64 x 1024 x 64)."""
    x, y, bias = _mk(m, k, n, dtype, k + n)
    xd, yd, bd = x.to(DEV), y.to(DEV), bias.to(DEV)
    lib = _lib.load()
    auto = lib.hx_matmul_splits(m, n, k, k, n, 1, n, _DT[dtype], 0)
    assert auto > 1
    ref = orc.matmul(x, y)
    refb = orc.matmul(x, y, bias, relu=True)
    for split in (0, 1, 2, 8, 1 << 20):
        out = hx.matmul_split_k(xd, yd, split_k=split)
        assert out.dtype == dtype and rel_err(out, ref) <= 1e-2
        outb = hx.matmul_split_k(xd, yd, bias_relu(bd), split_k=split)
        assert rel_err(outb, refb) <= 1e-2
    # fp32 partial sums in a fixed order: the same call twice is bit-identical (the reference's atomics are not)
    assert torch.equal(hx.matmul_split_k(xd, yd), hx.matmul_split_k(xd, yd))
    lam = hx.matmul_split_k(xd, yd, lambda acc, tile: acc + bd[tile[1]])
    assert rel_err(lam, orc.matmul(x, y, bias)) <= 1e-2


@pytest.mark.parametrize("m,k,n", [(3072, 256, 3072), (3000, 192, 3080)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_split_k_on_the_256_tile_kernel(m, k, n, dtype):
    """More than 128 tiles of 256 x 256: an explicit split_k then runs the 256 x 256 kernel's fp32 partial-sum mode
    (full and ragged edge tiles, row-major and column-major W), the reduction adds the epilogue."""
    x, y, bias = _mk(m, k, n, dtype, m + k + n)
    xd, yd, bd = x.to(DEV), y.to(DEV), bias.to(DEV)
    ref = orc.matmul(x, y)
    refb = orc.matmul(x, y, bias, relu=True)
    for yy in (yd, yd.t().contiguous().t()):
        out = hx.matmul_split_k(xd, yy, split_k=2)
        assert out.dtype == dtype and rel_err(out, ref) <= 1e-2
        assert rel_err(hx.matmul_split_k(xd, yy, bias_relu(bd), split_k=3), refb) <= 1e-2
        assert torch.equal(out, hx.matmul_split_k(xd, yy, split_k=2))


def test_strided_operands_and_tritonbench_wrappers():
    x, y, bias = _mk(300, 256, 264, torch.bfloat16, 11)
    xd, yd, bd = x.to(DEV), y.to(DEV), bias.to(DEV)
    ref = orc.matmul(x, y, bias)
    wide = torch.zeros(300, 512, dtype=torch.bfloat16, device=DEV); wide[:, :256] = xd
    assert rel_err(hx.matmul(wide[:, :256], yd, bias_add(bd)), ref) <= 1e-2        # lda > K: read in place
    yt = yd.t().contiguous().t()[:, ::2]                                            # strided in both dimensions: plain kernel
    assert rel_err(hx.matmul(xd, yt, bias_add(bd[::2])), orc.matmul(x, y[:, ::2], bias[::2])) <= 1e-2
    yt = yd.t().contiguous().t()                                                    # column-major y: tile kernel
    assert rel_err(hx.matmul(xd, yt, bias_add(bd)), ref) <= 1e-2
    assert rel_err(hx.matmul_tritonbench(xd, yd, bd)(), ref) <= 1e-2
    assert rel_err(hx.matmul_tritonbench(xd, yd, None)(), orc.matmul(x, y)) <= 1e-2
    assert rel_err(hx.matmul_split_k_tritonbench(xd, yd, bd)(), ref) <= 1e-2


def test_errors_and_empty():
    x = torch.zeros(4, 8, dtype=torch.float16, device=DEV)
    with pytest.raises(AssertionError):
        hx.matmul(x, torch.zeros(4, 8, dtype=torch.float16, device=DEV))
    with pytest.raises(TypeError):
        hx.matmul(x.to(torch.float64), x.t().to(torch.float64))
    with pytest.raises(ValueError):
        hx.matmul(x, x.t().contiguous(), bias_add(torch.zeros(3, dtype=torch.float16, device=DEV)))
    assert hx.matmul(x[:0], x.t()).shape == (0, 4)
    k0 = hx.matmul(torch.zeros(4, 0, dtype=torch.float16, device=DEV), torch.zeros(0, 8, dtype=torch.float16, device=DEV),
                   bias_add(torch.ones(8, dtype=torch.float16, device=DEV)))
    assert torch.equal(k0, torch.ones(4, 8, dtype=torch.float16, device=DEV))      # empty sum + bias


def test_golden_fixture():
    """Frozen oracle outputs (tests/golden/siblings_small.npz): an anchor that does not run the oracle code."""
    z = np.load(pathlib.Path(__file__).resolve().parent / "golden" / "siblings_small.npz")
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        t = lambda key: torch.from_numpy(z[key].copy()).view(dt)
        x, y, bias = (t(f"mm_{name}_{c}").to(DEV) for c in ("x", "y", "bias"))
        assert rel_err(hx.matmul(x, y), t(f"mm_{name}_out")) <= 1e-2
        assert rel_err(hx.matmul(x, y, bias_relu(bias)), t(f"mm_{name}_out_bias_relu")) <= 1e-2
