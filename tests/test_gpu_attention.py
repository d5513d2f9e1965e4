"""GPU parity of hx_fp8_attention against the CPU oracle (ref-eager semantics), the golden fixture,
closed-form cases, and at the benchmark size sampled heads plus key-permutation invariance."""
import pathlib

import numpy as np
import pytest
import torch

import helion_amd as hx
from helion_amd import _lib, inputs
from oracle import oracle as orc
from tests._util import TOL, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
# The online mode (exact_max=False) is NOT the parity mode: it restates the reference body with 64-key tiles, which is
# outside the 2e-2 bar against ref-eager by construction.  Against the 64-key tiled walk of the same lines it is
# asserted at 3e-2 (observed 3e-3 .. 2.1e-2): on top of the exact mode's P-rounding flips (the fp8 MFMA's inexact
# accumulation), a score that is the running maximum of its row moves the quantisation grid of everything after it.
TOL_ONLINE = 3e-2
E4M3 = torch.float8_e4m3fn
G = pathlib.Path(__file__).resolve().parent / "golden"


def _run(q, k, v, b, h, **kw):
    return hx.fp8_attention_kernel(q.to(DEV), k.to(DEV), v.to(DEV), b, h, **kw)


@pytest.mark.parametrize("b,h,s,d", [(1, 2, 128, 64), (2, 4, 256, 64), (4, 8, 512, 128),  # examples/fp8_attention.py:291-293
                                     (1, 1, 64, 64), (1, 3, 192, 128), (1, 9, 320, 128), (2, 5, 64, 128), (1, 1, 1024, 128)])
def test_exact_max_vs_oracle(b, h, s, d):
    q, k, v = inputs.attention_inputs(b, h, s, d, seed=s + d + h)
    ref32 = orc.fp8_attention(q, k, v, b, h, torch.float32)
    out32 = _run(q, k, v, b, h, out_dtype=torch.float32)
    assert out32.shape == (b, h, s, d)
    assert rel_err(out32, ref32) <= TOL
    out8 = _run(q, k, v, b, h)
    assert out8.dtype == E4M3
    ref8 = orc.fp8_attention(q, k, v, b, h)
    # after e4m3 output rounding a single differing code is 1/8..1/16 of that element; compare as values
    assert rel_err(out8, ref8) <= 0.08
    assert (out8.cpu().view(torch.uint8) == ref8.view(torch.uint8)).float().mean().item() > 0.98


@pytest.mark.parametrize("b,h,s,d", [(2, 4, 256, 64), (1, 2, 512, 128), (1, 3, 1024, 128), (1, 2, 333, 128), (2, 1, 200, 64)])
def test_online_mode_vs_the_tiled_oracle(b, h, s, d):
    """exact_max=False is the reference kernel body with its key loop in 64-key tiles (what the compiled kernel
    executes): parity bar against that walk of the same lines; against the one-tile (ref-eager) form it deviates by a
    few percent by construction (P is quantised against the running max)."""
    q, k, v = inputs.attention_inputs(b, h, s, d, seed=5)
    qd, kd = q.to(DEV), k.to(DEV)
    v_sd = v.to(DEV).transpose(1, 2).contiguous().transpose(1, 2)  # the layout the reference's preprocessing hands over
    out = hx.fp8_attention_kernel(qd, kd, v_sd, b, h, out_dtype=torch.float32, exact_max=False)
    assert rel_err(out, orc.fp8_attention_tiled(q, k, v, b, h, 64, torch.float32)) <= TOL_ONLINE
    assert rel_err(out, orc.fp8_attention(q, k, v, b, h, torch.float32)) <= 0.08


def test_golden_fixture():
    z = np.load(G / "fp8_attention_small.npz")
    for name in ("d64", "d128"):
        b, h, s, d = (int(x) for x in z[f"{name}_shape"])
        q, k, v = (torch.from_numpy(z[f"{name}_{t}"].copy()).view(E4M3) for t in "qkv")
        out = _run(q, k, v, b, h, out_dtype=torch.float32)
        assert rel_err(out, torch.from_numpy(z[f"{name}_out_f32"].copy())) <= TOL


def test_uniform_scores_give_mean_of_v_and_single_hot_key():
    s, d = 128, 128
    g = torch.Generator().manual_seed(6)
    q = torch.zeros(1, s, d).to(E4M3)
    k = torch.randn(1, s, d, generator=g).to(E4M3)
    v = torch.randn(1, d, s, generator=g).to(E4M3)
    out = _run(q, k, v, 1, 1, out_dtype=torch.float32)[0, 0].cpu()
    mean = orc.dq(v)[0].double().mean(1).float()
    assert torch.allclose(out, mean.expand(s, d), rtol=0, atol=2e-6)
    # one key dominates by a huge margin: output is that key's value row
    q2 = torch.zeros(1, s, d); k2 = torch.zeros(1, s, d)
    q2[0, :, 0] = 16.0; k2[0, 37, 0] = 448.0
    out2 = _run(q2.to(E4M3), k2.to(E4M3), v, 1, 1, out_dtype=torch.float32)[0, 0].cpu()
    # the kernel forms s*c - m with one rounding where the reference has two: with scores this large (2^10)
    # the winning key's p is 1 +- 2e-5 instead of exactly 1
    assert torch.allclose(out2, orc.dq(v)[0][:, 37].expand(s, d), rtol=1e-4, atol=1e-6)


def test_tritonbench_thunk_and_layout():
    torch.manual_seed(42)
    q, k, v = (torch.randn(2, 3, 128, 64, dtype=torch.float16) for _ in range(3))
    fn = hx.fp8_attention_tritonbench(q.to(DEV), k.to(DEV), v.to(DEV))
    out = fn()
    assert out.shape == (2, 3, 128, 64) and out.dtype == E4M3
    q8, k8, v8 = orc.preprocess_fp8_attention_inputs(q, k, v)
    assert rel_err(out, orc.fp8_attention(q8, k8, v8, 2, 3)) <= 0.08


def _path(qd, kd, vd):
    bh, s, d = qd.shape
    return _lib.load().hx_fp8_attention_path(bh, s, d, vd.stride(1), vd.stride(2), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), qd.data_ptr())


@pytest.mark.parametrize("b,h,s,d", [(1, 2, 100, 64), (1, 2, 16, 128), (1, 1, 48, 128), (2, 2, 80, 128), (2, 1, 333, 128), (1, 1, 400, 128),
                                     (1, 2, 1000, 64), (1, 2, 1100, 128), (1, 1, 7, 64), (1, 1, 1, 128), (1, 3, 4100, 128)])
def test_any_sequence_length_runs_the_mfma_kernel(b, h, s, d):
    """examples/fp8_attention.py:59,66 tile any seq_len.  The MFMA kernel masks a partial last key tile (and partial
    last query rows); both V layouts take it ([D][S] rows must be a multiple of 16 bytes to be fetched in place -
    otherwise the op hands the kernel the [S][D] order), both modes, both output types."""
    q, k, v = inputs.attention_inputs(b, h, s, d, seed=s + d)
    ref32 = orc.fp8_attention(q, k, v, b, h, torch.float32)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    v_sd = vd.transpose(1, 2).contiguous().transpose(1, 2)           # [BH, D, S] view of [BH, S, D] memory
    assert _path(qd, kd, v_sd) == 1
    if s > 1:
        assert _path(qd, kd, vd) == (1 if s % 16 == 0 else 0)
    assert rel_err(hx.fp8_attention_kernel(qd, kd, v_sd, b, h, out_dtype=torch.float32), ref32) <= TOL
    assert rel_err(hx.fp8_attention_kernel(qd, kd, vd, b, h, out_dtype=torch.float32), ref32) <= TOL
    out8 = hx.fp8_attention_kernel(qd, kd, v_sd, b, h)
    assert out8.dtype == E4M3 and rel_err(out8, orc.fp8_attention(q, k, v, b, h)) <= 0.08
    online = hx.fp8_attention_kernel(qd, kd, v_sd, b, h, out_dtype=torch.float32, exact_max=False)
    assert rel_err(online, orc.fp8_attention_tiled(q, k, v, b, h, 64, torch.float32)) <= TOL_ONLINE


@pytest.mark.parametrize("b,h,s,d", [(2, 1, 70, 80), (1, 3, 64, 32), (1, 1, 1, 16), (1, 1, 130, 256), (1, 2, 75, 200)])
def test_other_head_dims(b, h, s, d):
    """Head dims other than 64 / 128: up to 128 the op zero-pads onto the MFMA kernel, above that the plain kernel
    runs; exact-max form, both V layouts, both output types."""
    q, k, v = inputs.attention_inputs(b, h, s, d, seed=s + d)
    ref32 = orc.fp8_attention(q, k, v, b, h, torch.float32)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out = hx.fp8_attention_kernel(qd, kd, vd, b, h, out_dtype=torch.float32)
    assert rel_err(out, ref32) <= 2e-2
    v_sd = vd.transpose(1, 2).contiguous().transpose(1, 2)           # [BH, D, S] view of [BH, S, D] memory
    assert rel_err(hx.fp8_attention_kernel(qd, kd, v_sd, b, h, out_dtype=torch.float32), ref32) <= 2e-2
    out8 = hx.fp8_attention_kernel(qd, kd, vd, b, h)
    assert out8.dtype == E4M3 and rel_err(out8, orc.fp8_attention(q, k, v, b, h)) <= 0.08


@pytest.mark.parametrize("d", [32, 96])
def test_other_head_dims_are_zero_padded_onto_the_mfma_kernel(d):
    b, h, s = 1, 3, 256
    q, k, v = inputs.attention_inputs(b, h, s, d, seed=d)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out = hx.fp8_attention_kernel(qd, kd, vd, b, h, out_dtype=torch.float32)
    assert out.shape == (b, h, s, d) and out.is_contiguous()
    assert rel_err(out, orc.fp8_attention(q, k, v, b, h, torch.float32)) <= 2e-2
    v_sd = vd.transpose(1, 2).contiguous().transpose(1, 2)           # the [S][D] memory order
    assert rel_err(hx.fp8_attention_kernel(qd, kd, v_sd, b, h, out_dtype=torch.float32), orc.fp8_attention(q, k, v, b, h, torch.float32)) <= 2e-2
    out8 = hx.fp8_attention_kernel(qd, kd, vd, b, h)
    assert rel_err(out8, orc.fp8_attention(q, k, v, b, h)) <= 0.08


def test_unsupported_shapes_raise():
    x = torch.zeros(1, 64, 320).to(E4M3).to(DEV)
    with pytest.raises(ValueError, match="unsupported shape"):
        hx.fp8_attention_kernel(x, x, torch.zeros(1, 320, 64).to(E4M3).to(DEV), 1, 1)   # head dim > 256
    y = torch.zeros(2, 64, 64).to(E4M3).to(DEV)
    with pytest.raises(ValueError):
        hx.fp8_attention_kernel(y, y, y, 1, 1)  # batch*heads mismatch


def test_c4_sampled_heads_and_key_permutation():
    b, h, s, d = 4, 32, 4096, 128
    q, k, v = inputs.attention_c4()
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out = hx.fp8_attention_kernel(qd, kd, vd, b, h, out_dtype=torch.float32)
    # heads are mapped to XCDs by (head & 7): one head per XCD, among them the first and the last one
    for bh in (0, 9, 18, 27, 36, 77, 126, 127):
        ref = orc.fp8_attention(q[bh : bh + 1], k[bh : bh + 1], v[bh : bh + 1], 1, 1, torch.float32)
        assert rel_err(out[bh // h, bh % h], ref[0, 0]) <= TOL
    assert sorted({bh & 7 for bh in (0, 9, 18, 27, 36, 77, 126, 127)}) == list(range(8))
    # the online mode at full size against the 64-key tiled walk (two heads)
    online = hx.fp8_attention_kernel(qd, kd, vd, b, h, out_dtype=torch.float32, exact_max=False)
    for bh in (3, 100):
        reft = orc.fp8_attention_tiled(q[bh : bh + 1], k[bh : bh + 1], v[bh : bh + 1], 1, 1, 64, torch.float32)
        assert rel_err(online[bh // h, bh % h], reft[0, 0]) <= TOL_ONLINE
    perm = torch.randperm(s, generator=torch.Generator().manual_seed(1)).to(DEV)
    out_p = hx.fp8_attention_kernel(qd, kd[:, perm].contiguous(), vd[:, :, perm].contiguous(), b, h, out_dtype=torch.float32)
    # same exact row max, same quantisation grid; only MFMA summation order differs
    assert rel_err(out_p, out) <= 5e-3


@pytest.mark.parametrize("b,h,s,d", [(1, 2, 128, 64), (2, 3, 256, 64), (1, 3, 192, 128), (2, 4, 512, 128)])
@pytest.mark.parametrize("exact", [True, False])
def test_v_as_permuted_view_of_seq_major_memory(b, h, s, d, exact):
    """examples/fp8_attention.py:110-133 hands v over as a [BH, D, S] *view* of [BH, S, D] memory (permute, cast,
    reshape: strides (S*D, 1, D)).  The kernel reads that layout in place; operands and summation order are the
    same as for the contiguous [BH, D, S] tensor, so the results must be identical bit for bit."""
    g = torch.Generator().manual_seed(s + d)
    q32, k32, v32 = (torch.randn(b, h, s, d, generator=g) for _ in range(3))
    q8, k8, v8 = hx.preprocess_fp8_attention_inputs(q32.to(DEV), k32.to(DEV), v32.to(DEV))
    assert v8.shape == (b * h, d, s) and v8.stride() == (s * d, 1, d)       # what the reference's own code produces
    out_view = hx.fp8_attention_kernel(q8, k8, v8, b, h, out_dtype=torch.float32, exact_max=exact)
    out_contig = hx.fp8_attention_kernel(q8, k8, v8.contiguous(), b, h, out_dtype=torch.float32, exact_max=exact)
    assert torch.equal(out_view, out_contig)
    if exact:
        ref = orc.fp8_attention(q8.cpu(), k8.cpu(), v8.cpu(), b, h, torch.float32)
        assert rel_err(out_view, ref) <= TOL
        out8 = hx.fp8_attention_kernel(q8, k8, v8, b, h)
        assert torch.equal(out8.view(torch.uint8), hx.fp8_attention_kernel(q8, k8, v8.contiguous(), b, h).view(torch.uint8))


def test_tritonbench_wrapper_runs_on_the_reference_layout():
    g = torch.Generator().manual_seed(11)
    q32, k32, v32 = (torch.randn(1, 2, 256, 128, generator=g).to(DEV) for _ in range(3))
    out = hx.fp8_attention_tritonbench(q32, k32, v32)()
    q8, k8, v8 = hx.preprocess_fp8_attention_inputs(q32.cpu(), k32.cpu(), v32.cpu())
    ref = orc.fp8_attention(q8, k8, v8, 1, 2)
    assert out.dtype == E4M3 and rel_err(out, ref) <= 0.08


def test_random_shapes_layouts_vs_oracle():
    """A seeded sweep over head counts, sequence lengths (every multiple of 64 class: 64, odd multiples, multiples of
    128), both head dims, both V memory orders and both output types."""
    rng = np.random.default_rng(99)
    for case in range(20):
        b = int(rng.integers(1, 3)); h = int(rng.integers(1, 6))
        s = int(rng.choice([64, 128, 192, 320, 448, 512, 704, 90, 250, 1, 33]))
        d = int(rng.choice([64, 128]))
        v_seq_major = bool(rng.integers(0, 2))
        q, k, v = inputs.attention_inputs(b, h, s, d, seed=1000 + case)
        vd = v.to(DEV)
        if v_seq_major:
            vd = vd.transpose(1, 2).contiguous().transpose(1, 2)        # [BH, D, S] view of [BH, S, D] memory
            assert vd.stride() == (s * d, 1, d)
        ref = orc.fp8_attention(q, k, v, b, h, torch.float32)
        out = hx.fp8_attention_kernel(q.to(DEV), k.to(DEV), vd, b, h, out_dtype=torch.float32)
        assert rel_err(out, ref) <= TOL, (case, b, h, s, d, v_seq_major)
        out8 = hx.fp8_attention_kernel(q.to(DEV), k.to(DEV), vd, b, h)
        assert rel_err(out8, orc.fp8_attention(q, k, v, b, h)) <= 0.08, (case, b, h, s, d, v_seq_major)
        online = hx.fp8_attention_kernel(q.to(DEV), k.to(DEV), vd, b, h, out_dtype=torch.float32, exact_max=False)
        assert rel_err(online, orc.fp8_attention_tiled(q, k, v, b, h, 64, torch.float32)) <= TOL_ONLINE, (case, b, h, s, d, v_seq_major)
