"""GPU parity of the cast / quantise kernels in front of the FP8 kernels: bit-exact against torch's CPU cast (the
operation examples/fp8_attention.py:113-121 performs) and against the oracle's per-tensor quantiser."""
import numpy as np
import pytest
import torch

import helion_amd as hx
from helion_amd import ops
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"
E4M3 = torch.float8_e4m3fn


def _cast(x):
    return ops.cast_e4m3_x3_op(x.to(DEV), x.to(DEV), x.to(DEV))[1].cpu()


def _same_codes(got, want, src):
    """Equal byte for byte, except that for NaN sources any NaN code (0x7f / 0xff) is accepted."""
    g, w = got.view(torch.uint8), want.view(torch.uint8)
    nan_src = torch.isnan(src.float()).reshape(g.shape)
    assert torch.equal(g[~nan_src], w[~nan_src])
    assert bool(((g[nan_src] & 0x7F) == 0x7F).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cast_every_16_bit_pattern(dtype):
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    _same_codes(_cast(x), x.to(E4M3), x)


def test_cast_fp32_edges_and_random():
    g = torch.Generator().manual_seed(0)
    grid = torch.from_numpy(orc.E4M3_DECODE_TABLE[:127].astype(np.float32))           # every finite positive value
    mids = (grid[1:] + grid[:-1]) / 2                                                 # every rounding midpoint
    edge = torch.tensor([448.0, 463.9, 464.0, 464.1, 480.0, 1e9, float("inf"), float("nan"), 2.0 ** -9, 2.0 ** -10,
                         2.0 ** -10 * 1.0001, 0.0, -0.0, 1e-30])
    x = torch.cat([grid, mids, torch.nextafter(mids, torch.tensor(0.0)), torch.nextafter(mids, torch.tensor(1e9)), edge,
                   torch.randn(100000, generator=g) * 50, torch.randn(100000, generator=g) * 0.01])
    x = torch.cat([x, -x])
    _same_codes(_cast(x), x.to(E4M3), x)
    _same_codes(_cast(x), orc.to_e4m3(x), x)    # and against the closed-form encoder


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 4097, 1 << 20])
def test_cast_ragged_lengths(n):
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(n, generator=g) * 4).to(torch.bfloat16)
    _same_codes(_cast(x), x.to(E4M3), x)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_preprocess_matches_the_reference_function(dtype):
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(2, 3, 128, 64, generator=g).to(dtype) for _ in range(3))
    got = hx.preprocess_fp8_attention_inputs(q.to(DEV), k.to(DEV), v.to(DEV))
    want = orc.preprocess_fp8_attention_inputs(q, k, v)       # examples/fp8_attention.py:110-133 on the CPU
    for a, b in zip(got, want):
        assert a.shape == b.shape and a.stride() == b.stride() and a.dtype == E4M3
        assert torch.equal(a.cpu().view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape,scale", [((1,), 1.0), ((33,), 1e-3), ((256, 512), 7.0), ((1000, 1001), 300.0)])
def test_quantize_bit_exact_vs_oracle(dtype, shape, scale):
    g = torch.Generator().manual_seed(len(shape) + int(scale))
    x = (torch.randn(*shape, generator=g) * scale).to(dtype)
    q, s = hx.fp8_quantize_per_tensor(x.to(DEV))
    rq, rs = orc.fp8_quantize_per_tensor(x)
    assert q.shape == x.shape and q.dtype == E4M3 and s.dtype == torch.float32 and s.dim() == 0
    assert float(s) == float(rs)
    assert torch.equal(q.cpu().view(torch.uint8), rq.view(torch.uint8))


def test_quantize_zero_tensor_and_round_trip_through_the_scaled_gemm():
    q, s = hx.fp8_quantize_per_tensor(torch.zeros(64, 128, device=DEV))
    assert float(s) == 1.0 and bool((q.cpu().view(torch.uint8) == 0).all())
    g = torch.Generator().manual_seed(5)
    a = torch.randn(256, 256, generator=g) * 0.02
    b = torch.randn(256, 256, generator=g) * 5.0
    a8, sa = hx.fp8_quantize_per_tensor(a.to(DEV))
    b8, sb = hx.fp8_quantize_per_tensor(b.T.contiguous().to(DEV))      # B^T [N, K] row-major == column-major B
    out = hx.fp8_gemm_scaled(a8, b8.T, sa, sb, out_dtype=torch.float32).cpu()
    ref = a @ b
    assert float((out - ref).abs().max() / ref.abs().max()) < 0.05      # e4m3 quantisation noise, not a parity bound
    exact = (orc.dq(a8.cpu()) @ orc.dq(b8.cpu()).T) * float(sa) * float(sb)
    assert float((out - exact).abs().max() / exact.abs().max()) < 2e-3  # the kernel itself
