"""Pins oracle.fp8_gemm: float64 brute force (C restatement), bit-equality with the routine the reference
calls (CPU torch._scaled_mm, helion/language/matmul_ops.py:235-242) and with the literal ref-eager walk."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

E4M3 = torch.float8_e4m3fn


def _rand_fp8(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).clamp(-448, 448).to(E4M3)


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (7, 5, 3), (32, 32, 32), (17, 33, 65)])
def test_against_float64_bruteforce(oracle_c, m, n, k):
    x, y = _rand_fp8((m, k), 1), _rand_fp8((k, n), 2)
    yt = y.T.contiguous()
    out = np.empty((m, n), dtype=np.float64)
    xb, yb = x.view(torch.uint8).numpy().copy(), yt.view(torch.uint8).numpy().copy()
    oracle_c.orc_fp8_gemm_f64(xb.ctypes.data, yb.ctypes.data, out.ctypes.data, m, n, k)
    got = orc.fp8_gemm(x, y, out_dtype=torch.float32).double().numpy()
    # products are exact; only the fp32 summation rounds: relative 2^-24 per add
    assert np.allclose(got, out, rtol=0, atol=1e-6 * max(1.0, np.abs(out).max()) * k ** 0.5)
    # a transposed operand, a dropped k term or a wrong sign would be far outside this
    assert np.abs(out).max() > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bit_equal_to_cpu_scaled_mm(dtype):
    x, y = _rand_fp8((96, 160), 3), _rand_fp8((160, 64), 4)
    one = torch.tensor(1.0)
    lib = torch._scaled_mm(x, y.T.contiguous().T, one, one, use_fast_accum=False, out_dtype=dtype)
    assert torch.equal(orc.fp8_gemm(x, y, out_dtype=dtype), lib)
    assert torch.equal(orc.fp8_gemm_ref_eager(x, y, out_dtype=dtype), lib)


def test_scales_are_a_single_fp32_multiplier():
    x, y = _rand_fp8((8, 16), 5), _rand_fp8((16, 8), 6)
    sa, sb = torch.tensor(1.5), torch.tensor(0.75)
    base = orc.fp8_gemm(x, y, out_dtype=torch.float32)
    assert torch.equal(orc.fp8_gemm(x, y, sa, sb, torch.float32), base * (sa * sb))
    # linearity in the scale: doubling a scale doubles every element exactly (power of two)
    assert torch.equal(orc.fp8_gemm(x, y, sa * 2, sb, torch.float32), base * (sa * sb) * 2)


def test_identity_and_transpose_special_cases():
    eye = torch.eye(16).to(E4M3)
    y = _rand_fp8((16, 24), 7)
    assert torch.equal(orc.fp8_gemm(eye, y, out_dtype=torch.float32), orc.dq(y))
    x = _rand_fp8((24, 16), 8)
    assert torch.equal(orc.fp8_gemm(x, eye, out_dtype=torch.float32), orc.dq(x))
    # (x y)^T == y^T x^T exactly when sums are exact (small integers)
    xi = torch.randint(-3, 4, (5, 9), generator=torch.Generator().manual_seed(9)).float().to(E4M3)
    yi = torch.randint(-3, 4, (9, 4), generator=torch.Generator().manual_seed(10)).float().to(E4M3)
    a = orc.fp8_gemm(xi, yi, out_dtype=torch.float32)
    b = orc.fp8_gemm(yi.T.contiguous(), xi.T.contiguous(), out_dtype=torch.float32)
    assert torch.equal(a, b.T)
    assert torch.equal(a, xi.float() @ yi.float())


def test_default_output_dtype_is_fp16_like_the_reference():
    x, y = _rand_fp8((4, 8), 11), _rand_fp8((8, 4), 12)
    assert orc.fp8_gemm(x, y).dtype == torch.float16  # examples/fp8_gemm.py:46
