"""The host execution model (tests/sim) checked against itself and against the oracle's codec before any kernel result
obtained with it is believed: its e4m3 conversion is the oracle's over every rounding boundary, its operand buffers fault
on the first byte out of range, and each of its detection mechanisms (latest landing of DMA transfers, both wave
orders, guarded buffers) exposes the small defective kernel written for it while the correct form passes under every
variant."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.sim import simlib

E4 = torch.float8_e4m3fn


def test_fp8_conversion_is_the_oracles_on_every_code_midpoint_and_neighbour():
    lib = simlib.load()
    codes = np.arange(256, dtype=np.uint8)
    vals = orc.e4m3_decode(codes).astype(np.float64)
    pos = np.sort(vals[(codes < 0x7F)])  # 0 .. 448
    pts = [0.0, 1e-10, 2.0**-10, 2.0**-10 * 1.0001, 0.001, 448.0, 456.0, 463.99, 464.0, 464.01, 1000.0, float("inf"), float("nan")]
    for a, b in zip(pos[:-1], pos[1:]):
        mid = (a + b) / 2
        pts += [a, mid, np.nextafter(np.float32(mid), np.float32(0)), np.nextafter(np.float32(mid), np.float32(1e9))]
    x = np.array(pts, dtype=np.float32)
    x = np.concatenate([x, -x])
    want = torch.from_numpy(x).to(E4).view(torch.uint8).numpy()
    got = np.array([lib.hx_sim_cvt_pk_fp8(float(v), 0.0) & 0xFF for v in x], dtype=np.uint8)
    nan_w, nan_g = (want & 0x7F) == 0x7F, (got & 0x7F) == 0x7F
    assert (nan_w == nan_g).all()
    assert (want[~nan_w] == got[~nan_w]).all()
    # and it is the oracle's own encoder too
    enc = orc.e4m3_encode(x)
    assert (enc[~nan_w] == got[~nan_w]).all()


def _selftest(mode, variant, check_lds=True):
    lib = simlib.load()
    simlib.configure(variant)
    old = lib.hx_sim_set_check_lds(int(check_lds))
    try:
        return _selftest_run(lib, mode)
    finally:
        lib.hx_sim_set_check_lds(old)


def _selftest_run(lib, mode):
    with simlib.Arena() as ar:
        src = ar.put(torch.arange(4096, dtype=torch.int32).view(torch.uint8)[:4096].clone())
        dst = ar.out((4096,), torch.uint8, fill=0x11)
        rc = lib.hx_sim_selftest(src.data_ptr(), dst.data_ptr(), mode)
        fault = lib.hx_sim_last_fault().decode()
        lib.hx_sim_reset()
        return rc, fault, src.clone(), dst.clone()


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
def test_correct_protocol_passes_under_every_variant(variant):
    rc, fault, src, dst = _selftest(0, variant)
    assert rc == 0, fault
    assert torch.equal(src, dst)


def test_missing_wait_is_exposed_by_latest_landing():
    """Without the access check: invisible when transfers land at issue (as it mostly is on the hardware), a read of the
    poisoned LDS when they land as late as the wait allows."""
    rc, _, src, dst = _selftest(1, "eager", check_lds=False)
    assert rc == 0 and torch.equal(src, dst)
    rc, _, src, dst = _selftest(1, "lazy", check_lds=False)
    assert rc == 0 and not torch.equal(src, dst)
    assert bool((dst == 0xFF).all())


def test_missing_barrier_is_exposed_by_the_wave_order():
    want = torch.roll(_selftest(0, "eager")[2].reshape(4, 1024), -1, 0).reshape(-1)  # every wave copies the next one's data
    results = {v: torch.equal(_selftest(2, v, check_lds=False)[3], want) for v in ("eager", "lazy-reverse")}
    assert not all(results.values())  # at least one order reads a wave's data before that wave has fetched it


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
def test_lds_access_check_names_both_defects_under_every_variant(variant):
    """With the access check (the default) neither defect depends on the schedule to show: the read of bytes whose DMA
    has not been waited for, and the read of another wave's bytes without a barrier in between, stop the launch."""
    rc, fault, _, _ = _selftest(1, variant)
    assert rc != 0 and "LDS race" in fault and "DMA has not been waited for" in fault, fault
    rc, fault, _, _ = _selftest(2, variant)
    assert rc != 0 and "LDS race" in fault, fault


def test_a_read_one_byte_out_of_range_stops_the_launch_with_its_address():
    rc, fault, _, _ = _selftest(3, "lazy")
    assert rc != 0
    assert "out of bounds" in fault and "past the end of operand buffer 0" in fault


def test_a_fault_is_reported_not_fatal_and_the_next_launch_runs():
    _selftest(3, "eager")
    rc, fault, src, dst = _selftest(0, "eager")
    assert rc == 0 and torch.equal(src, dst), fault
