"""Pins oracle.fp8_attention against: the literal single-tile walk of the reference kernel body, a float64
brute force written independently in C, and closed-form special cases."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as orc

E4M3 = torch.float8_e4m3fn


def _inputs(b, h, s, d, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(b, h, s, d, generator=g).to(dtype) for _ in range(3))
    return orc.preprocess_fp8_attention_inputs(q, k, v)


def test_scale_constant_matches_the_golden_literal():
    # test/test_examples.expected:742-743 shows 0.18033688 for D=64
    assert float(orc.attention_scale(64)) == np.float32(0.18033688)
    assert float(orc.attention_scale(128)) == np.float32((1.0 / math.sqrt(128.0)) * 1.44269504)


@pytest.mark.parametrize("b,h,s,d", [(1, 2, 128, 64), (2, 2, 256, 64), (1, 1, 64, 128)])
def test_closed_form_equals_literal_walk(b, h, s, d):
    q, k, v = _inputs(b, h, s, d, 42, torch.float16)  # examples/fp8_attention.py:267-272 uses seed 42, fp16
    lit = orc.fp8_attention_literal(q, k, v, b, h)
    closed = orc.fp8_attention(q, k, v, b, h)
    assert torch.equal(lit.view(torch.uint8), closed.view(torch.uint8))
    assert not torch.isnan(closed.float()).any()


@pytest.mark.parametrize("s,d", [(8, 16), (32, 32), (16, 64)])
def test_against_float64_bruteforce(oracle_c, s, d):
    q, k, v = _inputs(1, 1, s, d, 3)
    out = np.empty((s, d), dtype=np.float32)
    qb, kb, vb = (t[0].contiguous().view(torch.uint8).numpy().copy() for t in (q, k, v))
    oracle_c.orc_fp8_attention_f64(qb.ctypes.data, kb.ctypes.data, vb.ctypes.data, out.ctypes.data, s, d)
    got = orc.fp8_attention(q, k, v, 1, 1, torch.float32)[0, 0].numpy()
    # identical quantisation points, only summation precision differs (an exp2 ulp can flip an e4m3 tie
    # in principle; none does for these seeds)
    assert np.abs(got - out).max() <= 2e-6 * max(1.0, np.abs(out).max())


def test_single_key_returns_v():
    d = 32
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 1, d, generator=g).to(E4M3)
    k = torch.randn(2, 1, d, generator=g).to(E4M3)
    v = torch.randn(2, d, 1, generator=g).to(E4M3)
    out = orc.fp8_attention(q, k, v, 1, 2, torch.float32)
    assert torch.equal(out[0, :, 0, :], orc.dq(v)[:, :, 0])  # p == 1, l == 1


def test_uniform_scores_give_mean_of_v():
    s, d = 16, 32
    q = torch.zeros(1, s, d).to(E4M3)  # all scores 0 -> p = 1 everywhere, exactly representable
    g = torch.Generator().manual_seed(6)
    k = torch.randn(1, s, d, generator=g).to(E4M3)
    v = torch.randn(1, d, s, generator=g).to(E4M3)
    out = orc.fp8_attention(q, k, v, 1, 1, torch.float32)[0, 0]
    mean = orc.dq(v)[0].double().mean(dim=1).float()
    assert torch.allclose(out, mean.expand(s, d), rtol=0, atol=1e-6)


def test_p_is_quantised_but_l_is_not():
    # two keys, scores chosen so p = [1, 2^-0.5]: e4m3(0.70710678) = 0.6875, l = 1.70710678
    d = 16
    q = torch.zeros(1, 1, d); k = torch.zeros(1, 2, d)
    q[0, 0, 0] = 2.0
    c = float(orc.attention_scale(d))
    # want (q.k1 - q.k0)*c = -0.5  ->  k1[0]-k0[0] = -0.25/c ; pick representable values by search
    cands = orc.E4M3_DECODE_TABLE[:0x7F]
    best = min(((abs((2.0 * float(a)) * c - 0.5), float(a)) for a in cands), key=lambda t: t[0])[1]
    k[0, 0, 0] = best
    v = torch.zeros(1, d, 2); v[0, :, 0] = 0.0; v[0, :, 1] = 1.0
    q8, k8, v8 = q.to(E4M3), k.to(E4M3), v.to(E4M3)
    s0 = np.float32(np.float32(2.0 * best) * np.float32(c))
    p1 = np.exp2(np.float32(0.0) - s0, dtype=np.float32)
    p1_q = float(orc.e4m3_decode(orc.e4m3_encode(np.array([p1], dtype=np.float32)))[0])
    expect = np.float32(p1_q) / (np.float32(1.0) + p1)
    out = orc.fp8_attention(q8, k8, v8, 1, 1, torch.float32)[0, 0, 0, 0].item()
    assert abs(out - float(expect)) <= 1e-7
    assert p1_q != float(p1)  # the case really exercises the quantisation


def test_key_permutation_invariance():
    q, k, v = _inputs(1, 1, 64, 32, 7)
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(8))
    a = orc.fp8_attention(q, k, v, 1, 1, torch.float32)
    b = orc.fp8_attention(q, k[:, perm], v[:, :, perm], 1, 1, torch.float32)
    assert torch.allclose(a, b, rtol=0, atol=2e-6)


def test_output_layout_batch_heads():
    q, k, v = _inputs(2, 3, 64, 16, 9)
    out = orc.fp8_attention(q, k, v, 2, 3, torch.float32)
    assert out.shape == (2, 3, 64, 16)
    one = orc.fp8_attention(q[4:5], k[4:5], v[4:5], 1, 1, torch.float32)
    assert torch.equal(out[1, 1], one[0, 0])  # bh = 4 -> b = 1, h = 1 (examples/fp8_attention.py:56-57)


# ---- the key loop in tiles (the compiled kernel's online softmax) ------------------------------------------------
@pytest.mark.parametrize("b,h,s,d", [(1, 2, 128, 64), (1, 1, 96, 32)])
def test_tiled_with_one_tile_is_the_ref_eager_form(b, h, s, d):
    q, k, v = _inputs(b, h, s, d, 7)
    for tile in (s, s + 5, 4 * s):
        a = orc.fp8_attention_tiled(q, k, v, b, h, tile)
        assert torch.equal(a.view(torch.uint8), orc.fp8_attention(q, k, v, b, h).view(torch.uint8))


def _tiled_f64(q, k, v, tile_n):
    """Independent re-derivation for one head: explicit loops over rows and tiles in float64, p rounded to e4m3 by the
    numpy encoder, exp2 arguments formed in fp32 exactly as the reference's fp32 tensors do."""
    s, d = q.shape
    qd, kd, vd = (orc.e4m3_decode(t.view(torch.uint8).numpy()).astype(np.float64) for t in (q, k, v))  # v: [d, s]
    c = np.float32((1.0 / math.sqrt(float(d))) * 1.44269504)
    out = np.zeros((s, d))
    for r in range(s):
        m, l, acc = -np.inf, 0.0, np.zeros(d)
        for n0 in range(0, s, tile_n):
            n1 = min(n0 + tile_n, s)
            sc = (np.array([np.dot(qd[r], kd[j]) for j in range(n0, n1)]).astype(np.float32) * c).astype(np.float32)
            m_new = max(m, float(sc.max()))
            p = np.exp2((sc - np.float32(m_new)).astype(np.float32).astype(np.float64))
            alpha = 0.0 if m == -np.inf else 2.0 ** float(np.float32(m) - np.float32(m_new))
            l = l * alpha + p.sum()
            p8 = orc.e4m3_decode(orc.e4m3_encode(p.astype(np.float32))).astype(np.float64)
            acc = acc * alpha + np.array([np.dot(p8, vd[j, n0:n1]) for j in range(d)])
            m = m_new
        out[r] = acc / l
    return out


@pytest.mark.parametrize("s,d,tile", [(48, 16, 16), (64, 32, 16), (40, 16, 16)])
def test_tiled_against_float64_rederivation(s, d, tile):
    q, k, v = _inputs(1, 1, s, d, 11)
    got = orc.fp8_attention_tiled(q, k, v, 1, 1, tile, torch.float32)[0, 0].numpy()
    want = _tiled_f64(q[0], k[0], v[0], tile)
    # same quantisation points; fp32 vs float64 sums (an exp2 ulp could flip an e4m3 tie; none does for this seed)
    assert np.abs(got - want).max() <= 5e-6 * max(1.0, np.abs(want).max())
    # and the tiling matters: it is not the single-tile result
    one = orc.fp8_attention(q, k, v, 1, 1, torch.float32)[0, 0].numpy()
    assert np.abs(got - one).max() > 1e-4


def test_tiled_is_tile_invariant_when_p_is_exact():
    s, d = 64, 32
    q = torch.zeros(1, s, d).to(E4M3)  # uniform scores: p == 1 in every tile, whatever the running max
    g = torch.Generator().manual_seed(6)
    k = torch.randn(1, s, d, generator=g).to(E4M3)
    v = torch.randn(1, d, s, generator=g).to(E4M3)
    a = orc.fp8_attention_tiled(q, k, v, 1, 1, 16, torch.float32)
    b = orc.fp8_attention(q, k, v, 1, 1, torch.float32)
    assert torch.allclose(a, b, rtol=0, atol=1e-6)


def test_tiled_rescale_path_against_the_closed_form_when_p_is_not_quantised(monkeypatch):
    """Pins the alpha path (l and acc rescaled when the running max moves) by mathematics rather than by a second
    statement of the recurrence: with the e4m3 cast of p taken out (here only, through a patch local to this test) the
    online recurrence is an exact re-association of softmax(scores) @ v, so for any tiling it must equal the closed form
    evaluated in float64 - and it must do so on rows whose maximum moves from tile to tile, where alpha != 1.  A dropped
    or inverted alpha, or one applied to only one of l and acc, fails this by orders of magnitude."""
    monkeypatch.setattr(orc, "to_e4m3", lambda x: x)  # p stays fp32 ...
    decode = orc.dq
    monkeypatch.setattr(orc, "dq", lambda t: t if t.dtype == torch.float32 else decode(t))  # ... and is used as it is
    s, d, tile = 96, 32, 16
    q, k, v = _inputs(1, 1, s, d, 21)
    qd, kd, vd = (orc.e4m3_decode(t[0].view(torch.uint8).numpy()).astype(np.float64) for t in (q, k, v))
    c = float(np.float32((1.0 / math.sqrt(float(d))) * 1.44269504))
    sc = qd @ kd.T * c
    # the running max must move in later tiles for most rows, or the test would not exercise alpha
    tile_of_max = sc.argmax(1) // tile
    first_tile_max = sc[:, :tile].max(1)
    moves = (sc.max(1) > first_tile_max + 0.5).sum()
    assert moves >= s // 2 and (tile_of_max > 0).sum() >= s // 2
    w = np.exp2(sc - sc.max(1, keepdims=True))
    want = (w @ vd.T) / w.sum(1, keepdims=True)
    for t in (tile, 32, 40):
        got = orc.fp8_attention_tiled(q, k, v, 1, 1, t, torch.float32)[0, 0].numpy().astype(np.float64)
        assert np.abs(got - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
    one = orc.fp8_attention_tiled(q, k, v, 1, 1, s, torch.float32)[0, 0].numpy().astype(np.float64)
    assert np.abs(one - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
