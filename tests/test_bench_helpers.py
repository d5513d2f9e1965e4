"""bench.py's host-side helpers: the roofline arithmetic, the rule that a recorded traffic figure is only reported for
the kernel sources it was recorded with, and the one-GPU rule.  Nothing here touches a GPU."""
import subprocess
import sys

import pytest

import bench

_T = {"median_ms": 0.5, "mean_ms": 0.51, "min_ms": 0.49, "max_ms": 0.55, "whole_region_mean_ms": 0.52, "timed_launches": 20,
      "warmup_launches": 5, "settle_launches": 40, "engine_clock_mhz": None}


def test_mfma_roofline_arithmetic():
    r = bench._mfma_roofline(2.0 * 8192**3, _T, bench.PEAK_FP8_TFLOPS, bench.FP8_FLOP_PER_CU_CLK, "k")
    assert r["bound"] == "mfma" and r["unit"] == "TFLOP/s" and r["peak"] == bench.PEAK_FP8_TFLOPS
    assert r["achieved"] == pytest.approx(2.0 * 8192**3 / 0.5e-3 / 1e12)
    assert r["frac"] == pytest.approx(r["achieved"] / r["peak"])
    assert r["traffic"] is None  # no profile named: nothing is made up
    assert r["algorithmic_flops_per_launch"] == 2.0 * 8192**3


def test_hbm_roofline_arithmetic():
    nbytes = 235929600  # the decode configuration: N*K + M*K + 2*M*N
    r = bench._hbm_roofline(nbytes, _T, "k")
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == bench.PEAK_HBM_GBS == 8000.0
    assert r["achieved"] == pytest.approx(nbytes / 0.5e-3 / 1e9)
    assert r["frac"] == pytest.approx(r["achieved"] / 8000.0)
    assert r["algorithmic_bytes_per_launch"] == float(nbytes)


def test_published_peaks():
    assert bench.PEAK_FP8_TFLOPS == 5000.0 and bench.PEAK_BF16_TFLOPS == 2500.0


def test_traffic_is_reported_only_for_the_sources_it_was_recorded_with(tmp_path, monkeypatch):
    root = tmp_path
    (root / "profiles").mkdir()
    (root / "helion_amd" / "csrc").mkdir(parents=True)
    (root / "helion_amd" / "csrc" / "k.hip").write_text("kernel v1")
    monkeypatch.setattr(bench, "ROOT", root)
    digest = bench._sources_digest(["k.hip"])
    (root / "profiles" / "hbm_traffic_fetch_write_size.txt").write_text(f"some text\ntraffic_bytes mykernel 12345 {digest} k.hip\n")
    value, src = bench._traffic("mykernel")
    assert value == 12345 and src["kernel_sources"] == ["k.hip"] and src["sources_sha256_16"] == digest
    assert bench._traffic("another") == (None, None)
    (root / "helion_amd" / "csrc" / "k.hip").write_text("kernel v2")  # the kernel changed: the old figure is not its traffic
    value, src = bench._traffic("mykernel")
    assert value is None and "changed" in src["note"]
    (root / "helion_amd" / "csrc" / "k.hip").unlink()                  # a source file that is gone never matches
    assert bench._traffic("mykernel")[0] is None


def test_counters_are_reported_only_for_the_sources_they_were_recorded_with(tmp_path, monkeypatch):
    root = tmp_path
    (root / "profiles").mkdir()
    (root / "helion_amd" / "csrc").mkdir(parents=True)
    (root / "helion_amd" / "csrc" / "k.hip").write_text("kernel v1")
    monkeypatch.setattr(bench, "ROOT", root)
    digest = bench._sources_digest(["k.hip"])
    (root / "profiles" / "sq_tcc_counters_all_kernels.txt").write_text(f"text\nkernel_counters mykernel 1929 0.758 {digest} k.hip\n")
    c = bench._counters("mykernel")
    assert c["clock_mhz"] == 1929.0 and c["mfma_busy"] == 0.758 and c["sources_sha256_16"] == digest
    assert bench._counters("another") is None
    (root / "helion_amd" / "csrc" / "k.hip").write_text("kernel v2")
    c = bench._counters("mykernel")
    assert c["clock_mhz"] is None and c["mfma_busy"] is None and "changed" in c["note"]


def test_roofline_carries_counters_and_no_probe_fields_by_default(tmp_path, monkeypatch):
    """Without --clock-probe no probe kernel runs: engine_clock_mhz stays null and no clock-relative peak is printed."""
    assert bench.CLOCK_PROBE is False
    r = bench._mfma_roofline(2.0 * 8192**3, _T, bench.PEAK_FP8_TFLOPS, bench.FP8_FLOP_PER_CU_CLK, "k", "fp8_gemm_tile256_c2")
    assert r["engine_clock_mhz"] is None
    assert "peak_at_achieved_clock" not in r and "frac_of_peak_at_achieved_clock" not in r
    assert "counters" in r  # a dict (current digest or the reason it is withheld)
    assert r["counters"] is None or "note" in r["counters"]


def test_recorded_counter_lines_are_well_formed():
    f = bench.ROOT / "profiles" / "sq_tcc_counters_all_kernels.txt"
    lines = [l.split() for l in f.read_text().splitlines() if l.startswith("kernel_counters ")]
    assert any(p[1] == "fp8_gemm_tile256_c2" for p in lines)
    for p in lines:
        assert 500 < float(p[2]) < 2600 and 0.0 <= float(p[3]) <= 1.0 and len(p[4]) == 16
        for src in p[5:]:
            assert (bench.ROOT / "helion_amd" / "csrc" / src).exists(), src


def test_headline_traffic_record_names_existing_sources():
    """Every recorded traffic line must name kernel source files that exist (whether its digest is current is the bench's
    business at run time)."""
    f = bench.ROOT / "profiles" / "hbm_traffic_fetch_write_size.txt"
    lines = [l.split() for l in f.read_text().splitlines() if l.startswith("traffic_bytes ")]
    assert any(p[1] == "fp8_gemm_tile256_c2" for p in lines)
    for p in lines:
        assert int(p[2]) > 0 and len(p[3]) == 16
        for src in p[4:]:
            assert (bench.ROOT / "helion_amd" / "csrc" / src).exists(), src


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(bench.ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
