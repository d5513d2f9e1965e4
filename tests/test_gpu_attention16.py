"""GPU parity of hx_attention (the 16-bit sibling of the fp8 attention: examples/attention.py of the reference) against
the CPU oracle, through the C ABI via the registered op.  Bar: max|out - ref| <= 2e-2 max|ref| after rounding to the
output dtype."""
import pathlib

import numpy as np
import pytest
import torch

import helion_amd as hx
from helion_amd import _lib
from oracle import oracle as orc
from tests._util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
_DT = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def _mk(shape_q, n, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    *lead, m, d = shape_q
    q = (torch.randn(*lead, m, d, generator=g) * scale).to(dtype)
    k = (torch.randn(*lead, n, d, generator=g) * scale).to(dtype)
    v = torch.randn(*lead, n, d, generator=g).to(dtype)
    return q, k, v


def _path(q, k):
    bh = q.numel() // (q.shape[-2] * q.shape[-1])
    return _lib.load().hx_attention_path(bh, q.shape[-2], k.shape[-2], q.shape[-1], _DT[q.dtype], q.data_ptr(), k.data_ptr(),
                                         k.data_ptr(), q.data_ptr())


@pytest.mark.parametrize("shape_q,n,path", [
    ((2, 4, 256, 64), 256, 1), ((1, 2, 128, 128), 128, 1), ((2, 3, 1024, 64), 512, 1),   # seq_q != seq_k: test_examples.py:358-372
    ((1, 3, 100, 128), 192, 1), ((3, 1, 64), 64, 1), ((9, 33, 64), 1024, 1), ((1, 1, 200, 128), 2048, 1),
    ((2, 2, 50, 64), 70, 1), ((1, 3, 130, 128), 1, 1), ((2, 1, 64, 128), 63, 1), ((2, 2, 33, 64), 1000, 1), ((1, 2, 40, 32), 64, 0), ((1, 1, 17, 80), 33, 0), ((2, 5, 256), 9, 0),
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_shapes_vs_oracle(shape_q, n, path, dtype):
    q, k, v = _mk(shape_q, n, dtype, sum(shape_q) + n)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    assert _path(qd, kd) == path
    out = hx.attention(qd, kd, vd)
    assert out.dtype == dtype and out.shape == q.shape
    assert rel_err(out, orc.attention(q, k, v)) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_peaked_softmax_and_running_max_updates(dtype):
    """Large score spread: the running max keeps moving across key tiles and most probabilities underflow."""
    q, k, v = _mk((1, 2, 128, 64), 512, dtype, 7, scale=4.0)
    out = hx.attention(q.to(DEV), k.to(DEV), v.to(DEV))
    assert rel_err(out, orc.attention(q, k, v)) <= 2e-2
    # keys sorted so that every tile raises the max of some rows: same answer as any other key order
    perm = torch.argsort((q[0, 0, 0].float() @ k[0, 0].float().T))
    out_p = hx.attention(q.to(DEV), k[:, :, perm].to(DEV), v[:, :, perm].to(DEV))
    assert rel_err(out_p, orc.attention(q, k, v)) <= 2e-2


@pytest.mark.parametrize("d", [32, 80, 96, 112])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_other_head_dims_are_zero_padded_onto_the_mfma_kernel(d, dtype):
    """Head dims below 128 other than 64: the op pads q, k, v with zero columns and passes the true head dim for the
    softmax scale; same result as the oracle on the unpadded tensors, and as sdpa."""
    q, k, v = _mk((2, 3, 150, d), 200, dtype, d)
    out = hx.attention(q.to(DEV), k.to(DEV), v.to(DEV))
    assert out.shape == q.shape and out.is_contiguous()
    assert rel_err(out, orc.attention(q, k, v)) <= 2e-2
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert rel_err(out, want.to(dtype)) <= 2e-2


def test_fp32_inputs_and_sdpa_relation():
    """test/test_examples.py:342-356,374-388 feed fp32 tensors of shape (1, 32, 512, 64): plain kernel."""
    q, k, v = _mk((1, 4, 128, 64), 128, torch.float32, 11)
    out = hx.attention(q.to(DEV), k.to(DEV), v.to(DEV))
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), orc.attention(q, k, v), atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(out.cpu(), torch.nn.functional.scaled_dot_product_attention(q, k, v), atol=1e-4, rtol=1e-3)
    assert hx.attention_dynamic is hx.attention


def test_special_cases():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(2, 128, 64, generator=g).half().to(DEV)
    v = torch.randn(2, 64, 64, generator=g).half().to(DEV)
    k0 = torch.zeros(2, 64, 64, dtype=torch.float16, device=DEV)
    want = (v.float().sum(1, keepdim=True) / 64).half().expand(2, 128, 64)           # uniform scores: mean of v
    assert (hx.attention(q, k0, v).float() - want.float()).abs().max() <= 2e-3
    big = hx.attention(q, q[:, :64] * 0 + 0, v)                                       # same through a non-trivial expression
    assert torch.equal(big, hx.attention(q, k0, v))


def test_non_contiguous_inputs_and_errors():
    q, k, v = _mk((2, 2, 128, 64), 128, torch.bfloat16, 13)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    ref = orc.attention(q, k, v)
    kt = kd.transpose(-1, -2).contiguous().transpose(-1, -2)                        # same values, other strides
    assert rel_err(hx.attention(qd, kt, vd), ref) <= 2e-2
    with pytest.raises(TypeError):
        hx.attention(qd, kd.half(), vd)
    with pytest.raises(AssertionError):
        hx.attention(qd, kd[..., :64, :], vd)
    with pytest.raises(ValueError):
        hx.attention(qd, kd[:, :, :0], vd[:, :, :0])


def test_seeded_random_sweep():
    g = torch.Generator().manual_seed(99)
    for _ in range(12):
        d = (64, 128)[int(torch.randint(0, 2, (1,), generator=g))]
        bh = int(torch.randint(1, 20, (1,), generator=g)); m = int(torch.randint(1, 400, (1,), generator=g))
        n = int(torch.randint(1, 700, (1,), generator=g))
        dtype = (torch.float16, torch.bfloat16)[int(torch.randint(0, 2, (1,), generator=g))]
        q, k, v = _mk((bh, m, d), n, dtype, int(torch.randint(0, 1 << 30, (1,), generator=g)))
        out = hx.attention(q.to(DEV), k.to(DEV), v.to(DEV))
        assert rel_err(out, orc.attention(q, k, v)) <= 2e-2, (bh, m, n, d, dtype)


def test_golden_fixture():
    """Frozen oracle outputs (tests/golden/siblings_small.npz): an anchor that does not run the oracle code."""
    z = np.load(pathlib.Path(__file__).resolve().parent / "golden" / "siblings_small.npz")
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        t = lambda key: torch.from_numpy(z[key].copy()).view(dt)
        for tag in ("d64", "d128"):
            q, k, v = (t(f"att_{name}_{tag}_{c}").to(DEV) for c in "qkv")
            assert rel_err(hx.attention(q, k, v), t(f"att_{name}_{tag}_out")) <= 2e-2
