"""Pins oracle.matmul (the eager-mode restatement of examples/matmul.py:25-56 and examples/matmul_split_k.py:30-68)
without retyping its formula: float64 brute force with explicit loops, special cases with known answers, and the
relations the reference's own tests assert."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m,k,n", [(3, 5, 4), (8, 16, 8), (1, 7, 1)])
def test_brute_force_float64(dtype, m, k, n):
    g = torch.Generator().manual_seed(m * 100 + k * 10 + n)
    x = torch.randn(m, k, generator=g).to(dtype); y = torch.randn(k, n, generator=g).to(dtype)
    bias = torch.randn(n, generator=g).to(dtype)
    xs, ys, bs = x.double().numpy(), y.double().numpy(), bias.double().numpy()
    for use_bias, relu in ((False, False), (True, False), (True, True), (False, True)):
        want = np.zeros((m, n))
        for i in range(m):
            for j in range(n):
                s = 0.0
                for kk in range(k):
                    s += xs[i, kk] * ys[kk, j]
                if use_bias:
                    s += bs[j]
                want[i, j] = max(s, 0.0) if relu else s
        got = orc.matmul(x, y, bias if use_bias else None, relu)
        assert got.dtype == dtype and got.shape == (m, n)
        # the oracle sums in fp32 and rounds once to the output type: within one output ulp (of the magnitude of the
        # terms summed) of the float64 value
        eps = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2.0 ** -20}[dtype]
        mag = np.abs(xs) @ np.abs(ys) + (np.abs(bs) if use_bias else 0.0)
        assert np.all(np.abs(got.double().numpy() - want) <= eps * np.maximum(mag, 1.0))


def test_identity_and_zero_cases():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(16, 16, generator=g).half()
    eye = torch.eye(16).half()
    assert torch.equal(orc.matmul(x, eye), x)                      # x @ I = x exactly
    assert torch.equal(orc.matmul(eye, x), x)
    bias = torch.randn(16, generator=g).half()
    zero = torch.zeros(16, 16).half()
    assert torch.equal(orc.matmul(zero, x, bias), bias.expand(16, 16))          # 0 @ y + bias = bias in every row
    assert torch.equal(orc.matmul(zero, x, bias, relu=True), torch.relu(bias).expand(16, 16))
    assert torch.equal(orc.matmul(x, eye, relu=True), torch.relu(x))


def test_relations_the_reference_tests_assert():
    # test/test_examples.py:33-46 (x @ y, fp32), :143-200 (relu(x @ y + bias), fp16), :460-474 (split-K vs matmul)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(128, 128, generator=g); y = torch.randn(128, 128, generator=g)
    torch.testing.assert_close(orc.matmul(x, y), x @ y, atol=1e-4, rtol=1e-5)
    xh, yh = x.half(), y.half()
    bias = torch.randn(1, 128, generator=g).half()
    want = torch.relu(xh.float() @ yh.float() + bias.float()).half()
    torch.testing.assert_close(orc.matmul(xh, yh, bias, relu=True), want, atol=1e-2, rtol=1e-2)


def test_mixed_dtypes_promote():
    x = torch.ones(4, 4, dtype=torch.float16); y = torch.ones(4, 4, dtype=torch.float32)
    assert orc.matmul(x, y).dtype == torch.float32
    assert orc.matmul(x.bfloat16(), y.bfloat16(), out_dtype=torch.float32).dtype == torch.float32
