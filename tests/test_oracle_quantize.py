"""The oracle's per-tensor quantiser (the build's own definition; the reference only passes unit scales) pinned by
properties a wrong formula would break, and by the closed-form numpy e4m3 encoder."""
import numpy as np
import torch

from oracle import oracle as orc


def test_amax_element_lands_on_448_and_scale_is_amax_over_448():
    g = torch.Generator().manual_seed(0)
    for n in (1, 7, 1000):
        x = torch.randn(n, generator=g) * 3.7
        q, scale = orc.fp8_quantize_per_tensor(x)
        i = int(x.abs().argmax())
        assert abs(float(orc.dq(q)[i])) == 448.0
        assert float(scale) == float(x.abs().max() / torch.tensor(448.0))


def test_dequantised_value_is_within_half_a_step():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4096, generator=g)
    q, scale = orc.fp8_quantize_per_tensor(x)
    y = x / scale                      # what was rounded (up to one fp32 rounding)
    d = orc.dq(q)
    # e4m3 spacing at |y| in [2^e, 2^(e+1)) is 2^(e-3) (normal range), 2^-9 below 2^-6
    e = torch.floor(torch.log2(y.abs().clamp_min(2.0 ** -6)))
    half_step = torch.pow(2.0, e - 3) / 2
    assert bool(((d - y).abs() <= half_step * 1.0001 + 1e-6).all())


def test_power_of_two_scaling_changes_only_the_scale():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(513, generator=g)
    q1, s1 = orc.fp8_quantize_per_tensor(x)
    q2, s2 = orc.fp8_quantize_per_tensor(x * 8.0)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and float(s2) == float(s1) * 8.0


def test_zero_tensor_and_sign_symmetry():
    q, s = orc.fp8_quantize_per_tensor(torch.zeros(5))
    assert float(s) == 1.0 and bool((orc.dq(q) == 0).all())
    x = torch.tensor([0.3, -1.0, 0.77, 2.5])
    qa, _ = orc.fp8_quantize_per_tensor(x)
    qb, _ = orc.fp8_quantize_per_tensor(-x)
    assert torch.equal(orc.dq(qa), -orc.dq(qb))


def test_agrees_with_the_closed_form_numpy_encoder():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2000, generator=g) * 0.01
    q, scale = orc.fp8_quantize_per_tensor(x)
    inv = np.float32(448.0) / np.float32(x.abs().max())
    codes = orc.e4m3_encode((x.numpy().astype(np.float32) * inv).astype(np.float32))
    assert np.array_equal(codes, q.view(torch.uint8).numpy())
