"""Pins the oracle's e4m3fn codec: closed-form table vs torch's cast (the routine the reference uses,
examples/fp8_gemm.py:106-108, examples/fp8_attention.py:94) and vs the independent C restatement."""
import numpy as np
import torch

from oracle import oracle as orc


def test_decode_table_matches_torch_for_all_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    via_torch = codes.view(torch.float8_e4m3fn).float().numpy()
    ours = orc.e4m3_decode(codes.numpy())
    assert np.array_equal(np.isnan(via_torch), np.isnan(ours))
    ok = ~np.isnan(ours)
    assert np.array_equal(via_torch[ok], ours[ok])
    # spot values fixed by the format definition
    assert ours[0x38] == 1.0 and ours[0x7E] == 448.0 and ours[0x01] == 2.0**-9 and ours[0x08] == 2.0**-6
    assert ours[0xB8] == -1.0 and np.isnan(ours[0x7F]) and np.isnan(ours[0xFF])


def _probe_values():
    vals = orc.E4M3_DECODE_TABLE[:0x7F].astype(np.float32)
    pts = [vals]
    mids = (vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2
    mids = mids.astype(np.float32)  # exactly representable
    pts += [mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))]
    pts += [np.nextafter(vals, np.float32(0)), np.nextafter(vals, np.float32(1e9))]
    pts += [np.array([449, 463.99, 464, 464.0001, 465, 480, 1000, 1e30, np.inf, np.nan, 2.0**-10, 2.0**-11, 1e-10, 0.001],
                     dtype=np.float32)]
    rng = np.random.default_rng(0)
    pts += [np.ldexp(rng.random(200000), rng.integers(-12, 10, 200000)).astype(np.float32)]
    x = np.concatenate(pts)
    return np.concatenate([x, -x])


def test_encode_matches_torch_cast_on_midpoints_and_random():
    x = _probe_values()
    ours = orc.e4m3_encode(x)
    via_torch = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # NaN payload sign is irrelevant; compare modulo the sign of NaN codes
    nan_t = (via_torch & 0x7F) == 0x7F
    nan_o = (ours & 0x7F) == 0x7F
    assert np.array_equal(nan_t, nan_o)
    assert np.array_equal(ours[~nan_o], via_torch[~nan_o])


def test_encode_decode_roundtrip_is_identity_on_codes():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    back = orc.e4m3_encode(orc.e4m3_decode(codes))
    # -0 and +0 both decode to 0; everything else round-trips
    nz = (codes & 0x7F) != 0
    assert np.array_equal(back[nz], codes[nz])


def test_c_restatement_agrees(oracle_c):
    for c in range(256):
        a, b = oracle_c.orc_e4m3_decode(c), orc.E4M3_DECODE_TABLE[c]
        assert (np.isnan(a) and np.isnan(b)) or a == b
    x = _probe_values()[::7]
    ours = orc.e4m3_encode(x)
    theirs = np.array([oracle_c.orc_e4m3_encode(float(v)) for v in x], dtype=np.uint8)
    nan_o = (ours & 0x7F) == 0x7F
    assert np.array_equal(nan_o, (theirs & 0x7F) == 0x7F)
    assert np.array_equal(ours[~nan_o], theirs[~nan_o])
