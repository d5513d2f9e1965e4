"""The fp8 attention kernels executed on the CPU in the host execution model (tests/sim) against the oracle: both modes,
both memory layouts of V, both head dims, both output types, whole and ragged sequences incl. the lengths at which the
pipeline changes shape (first / steady-state / tail rounds of pass 1, branch-free and guarded steps of pass 2), operands
in guarded buffers, every scheduling / DMA-landing variant on one case.  The exact mode is held to the ref-eager oracle,
the online mode to the oracle that walks the key loop in 64-key tiles (it is the same recurrence: agreement is to fp32
rounding there, and by construction only to a few percent against the ref-eager form)."""
import pytest
import torch

from oracle import oracle as orc
from tests._util import attention_close, rel_err
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn


def _qkv(bh, s, d, seed):
    g = torch.Generator().manual_seed(seed)
    q, k = (torch.randn(bh, s, d, generator=g).to(E4) for _ in range(2))
    v = torch.randn(bh, d, s, generator=g).to(E4)
    return q, k, v


def _check(q, k, v, exact, layout, out_dtype=torch.float32, end_flush=True):
    bh = q.shape[0]
    out = simops.fp8_attention(q, k, v, 1, bh, out_dtype, exact, layout, end_flush=end_flush, want_path=1)
    if exact:
        ref = orc.fp8_attention(q, k, v, 1, bh, out_dtype)
    else:
        ref = orc.fp8_attention_tiled(q, k, v, 1, bh, 64, out_dtype)
    if out_dtype == torch.float32:
        assert not torch.isnan(out).any()
        assert attention_close(out, ref), (q.shape, exact, layout, rel_err(out, ref))
    else:  # e4m3 output: the same fp32 values rounded; allow a handful of one-code differences from summation order
        same = (out.view(torch.uint8) == ref.view(torch.uint8)).float().mean().item()
        assert same >= 0.999 and rel_err(orc.dq(out), orc.dq(ref)) <= 0.13, (q.shape, exact, layout, same)


# ntiles = ceil(S / 64): 1 .. 4 (prologue shapes), 8 / 9 (pass 1 switches to its steady-state rounds from 9 whole tiles
# + a tile, i.e. last >= 8), 10, 17 (two steady-state round pairs), ragged neighbours of each; the [D][S] layout needs S % 16 == 0
@pytest.mark.parametrize("s", [64, 128, 192, 208, 256, 320, 512, 560, 576, 592, 640, 1040, 1088])
@pytest.mark.parametrize("exact", [True, False])
def test_sequence_lengths_d128(s, exact):
    q, k, v = _qkv(1, s, 128, s)
    simlib.configure("lazy-reverse")
    _check(q, k, v, exact, "DS")
    simlib.configure("eager-interleaved")
    _check(q, k, v, exact, "SD")


@pytest.mark.parametrize("s", [1, 5, 63, 65, 100, 127, 129, 300, 777])
def test_sequence_lengths_not_a_multiple_of_16_take_the_strided_layout(s):
    q, k, v = _qkv(2, s, 64, s)
    simlib.configure("lazy")
    _check(q, k, v, True, "SD")
    _check(q, k, v, False, "SD")


@pytest.mark.parametrize("d,out_dtype", [(64, torch.float32), (64, E4), (128, E4)])
@pytest.mark.parametrize("layout", ["DS", "SD"])
def test_head_dims_and_output_types(d, out_dtype, layout):
    q, k, v = _qkv(3, 336, d, d)  # 3 heads: the head -> XCD mapping leaves five of eight workgroup slots empty
    simlib.configure("lazy-interleaved")
    _check(q, k, v, True, layout, out_dtype)
    _check(q, k, v, False, layout, out_dtype)


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
@pytest.mark.parametrize("exact", [True, False])
def test_every_variant(variant, exact):
    q, k, v = _qkv(1, 1104, 128, 7)  # 18 tiles, the last one partial: every loop shape of both passes
    simlib.configure(variant)
    _check(q, k, v, exact, "DS")


def test_operands_against_the_leading_page_too():
    q, k, v = _qkv(2, 400, 128, 11)
    simlib.configure("lazy")
    for layout in ("DS", "SD"):
        for exact in (True, False):
            _check(q, k, v, exact, layout, end_flush=False)


def test_plain_kernel_for_other_head_dims():
    g = torch.Generator().manual_seed(5)
    q, k = (torch.randn(2, 50, 40, generator=g).to(E4) for _ in range(2))
    v = torch.randn(2, 40, 50, generator=g).to(E4)
    simlib.configure("lazy")
    out = simops.fp8_attention(q, k, v, 1, 2, torch.float32, True, "DS", want_path=0)
    assert attention_close(out, orc.fp8_attention(q, k, v, 1, 2, torch.float32))


# ---- opt-in: head dim 256 on the MFMA kernel (HX_FEATURE_ATTENTION_D256) ------------------------------------------------
@pytest.mark.parametrize("s", [64, 208, 640, 1104])
@pytest.mark.parametrize("exact", [True, False])
def test_head_dim_256(s, exact):
    from helion_amd import _lib
    q, k, v = _qkv(1, s, 256, s)
    with simlib.features(_lib.HX_FEATURE_ATTENTION_D256):
        simlib.configure("lazy-reverse")
        _check(q, k, v, exact, "DS")
        simlib.configure("eager-interleaved")
        _check(q, k, v, exact, "SD", end_flush=False)


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
def test_head_dim_256_every_variant_and_e4m3_output(variant):
    from helion_amd import _lib
    q, k, v = _qkv(2, 331, 256, 3)
    simlib.configure(variant)
    with simlib.features(_lib.HX_FEATURE_ATTENTION_D256):
        _check(q, k, v, True, "SD", E4)
        _check(q, k, v, False, "SD")


def test_head_dim_256_is_the_plain_kernel_by_default():
    q, k, v = _qkv(1, 48, 256, 1)
    simlib.configure("lazy")
    out = simops.fp8_attention(q, k, v, 1, 1, torch.float32, True, "DS", want_path=0)
    assert attention_close(out, orc.fp8_attention(q, k, v, 1, 1, torch.float32))
