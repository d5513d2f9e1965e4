"""Pins oracle.attention (eager-mode restatement of examples/attention.py:33-84): float64 brute force with explicit
loops, closed-form special cases, invariances, and the relation the reference's tests assert."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2), (torch.float32, 1e-5)])
def test_brute_force_float64(dtype, tol):
    g = torch.Generator().manual_seed(3)
    B, M, N, D = 2, 5, 7, 8
    q = torch.randn(B, M, D, generator=g).to(dtype); k = torch.randn(B, N, D, generator=g).to(dtype)
    v = torch.randn(B, N, D, generator=g).to(dtype)
    qs, ks, vs = q.double().numpy(), k.double().numpy(), v.double().numpy()
    want = np.zeros((B, M, D))
    for b in range(B):
        for i in range(M):
            s = [sum(qs[b, i, d] * ks[b, j, d] for d in range(D)) / math.sqrt(D) for j in range(N)]
            mx = max(s)
            e = [math.exp(x - mx) for x in s]
            z = sum(e)
            for d in range(D):
                want[b, i, d] = sum(e[j] / z * vs[b, j, d] for j in range(N))
    got = orc.attention(q, k, v)
    assert got.dtype == dtype and got.shape == q.shape
    # differences: p is rounded to the value dtype before the P.V product, the output once more
    assert np.max(np.abs(got.double().numpy() - want)) <= tol * np.max(np.abs(want))


def test_special_cases_with_known_answers():
    g = torch.Generator().manual_seed(4)
    q = torch.randn(3, 6, 16, generator=g).half()
    v1 = torch.randn(3, 1, 16, generator=g).half(); k1 = torch.randn(3, 1, 16, generator=g).half()
    assert torch.equal(orc.attention(q, k1, v1), v1.expand(3, 6, 16))          # one key: softmax = 1, out = v
    k0 = torch.zeros(3, 8, 16).half()                                          # uniform scores: out = mean(v), p = 1 exactly
    v = torch.randn(3, 8, 16, generator=g).half()
    want = (v.float().sum(1, keepdim=True) / 8).half().expand(3, 6, 16)
    assert torch.equal(orc.attention(q, k0, v), want)
    # a dominant key: scores 0 everywhere but +huge at key 2 -> out = v[2]
    qd = torch.zeros(1, 2, 16).half(); qd[..., 0] = 60.0
    kd = torch.zeros(1, 4, 16).half(); kd[0, 2, 0] = 60.0
    vd = torch.randn(1, 4, 16, generator=g).half()
    assert torch.equal(orc.attention(qd, kd, vd), vd[:, 2:3].expand(1, 2, 16))


def test_key_permutation_invariance_and_shapes():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 4, 9, 32, generator=g).bfloat16()
    k = torch.randn(2, 4, 12, 32, generator=g).bfloat16(); v = torch.randn(2, 4, 12, 32, generator=g).bfloat16()
    a = orc.attention(q, k, v)
    assert a.shape == (2, 4, 9, 32)
    perm = torch.randperm(12, generator=g)
    b = orc.attention(q, k[:, :, perm], v[:, :, perm])
    assert (a.float() - b.float()).abs().max() <= 2 ** -7 * a.float().abs().max()   # summation order only


@pytest.mark.parametrize("dtype,atol", [(torch.float32, 1e-5), (torch.float16, 2e-3)])
def test_matches_sdpa_as_the_reference_tests_assert(dtype, atol):
    # test/test_examples.py:342-390: attention vs torch.nn.functional.scaled_dot_product_attention,
    # also with different query and key lengths
    g = torch.Generator().manual_seed(6)
    q = torch.randn(1, 4, 64, 64, generator=g).to(dtype)
    k = torch.randn(1, 4, 32, 64, generator=g).to(dtype); v = torch.randn(1, 4, 32, 64, generator=g).to(dtype)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    torch.testing.assert_close(orc.attention(q, k, v).float(), want, atol=atol, rtol=1e-2)
