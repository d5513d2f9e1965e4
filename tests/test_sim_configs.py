"""The BASELINE configurations in the host execution model (tests/sim), as far as a default test run can afford: C1 whole
(the reference's own CPU case, 1024^3), and the others with their real row / key / k dimensions and a slice of the
dimension the kernels treat independently (columns for the GEMMs, heads and query tiles for attention).  The full-size
runs are tests/sim/run_configs.py (minutes to an hour each; their results are recorded in the design document)."""
import torch

from helion_amd import inputs
from oracle import oracle as orc
from tests._util import attention_close, rel_err
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn


def test_c1_whole_output_bit_for_bit():
    a, b = inputs.gemm_c1()
    simlib.configure("lazy")
    out = simops.fp8_gemm(a, b, None, None, torch.bfloat16)
    ref = orc.fp8_gemm(a, b, 1.0, 1.0, torch.bfloat16)  # (bit-equal to the ref-eager form: tests/test_oracle_gemm.py)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_c2_full_k_a_band_of_the_output():
    """C2's K (8192: 64 k-tiles) and scales on a 512 x 1024 band.  (At this size the library picks its 128-column tiles; the
    256x256 kernel at the full 8192^3 - 1024 workgroups - is tests/sim/run_configs.py, and with 1 / 2 / 3 / 5 k-tiles
    tests/test_sim_fp8_gemm.py.)"""
    a, b, sa, sb = inputs.gemm_scaled(512, 1024, 8192, 1)
    simlib.configure("lazy-reverse")
    out = simops.fp8_gemm(a, b, sa, sb, torch.bfloat16, want_path=5)
    assert rel_err(out, orc.fp8_gemm(a, b, sa, sb, torch.bfloat16)) <= 1e-2


def test_c3_decode_kernel_full_k_an_eighth_of_the_columns():
    a, b, sa, sb = inputs.gemm_scaled(16, 28672 // 8, 8192, 2)
    simlib.configure("lazy")
    out = simops.fp8_gemm(a, b, sa, sb, torch.bfloat16, want_path=2)
    assert rel_err(out, orc.fp8_gemm(a, b, sa, sb, torch.bfloat16)) <= 1e-2


def test_c4_one_whole_head_per_mode():
    """One whole head at C4's sequence length and head dim (4096 queries x 4096 keys: 32 workgroups of 64 key tiles, the steady
    state of both passes), both modes."""
    q, k, v = inputs.attention_inputs(1, 1, 4096, 128, 3)
    simlib.configure("lazy")
    for exact in (True, False):
        out = simops.fp8_attention(q, k, v, 1, 1, torch.float32, exact, "DS", want_path=1)
        ref = orc.fp8_attention(q, k, v, 1, 1, torch.float32) if exact else orc.fp8_attention_tiled(q, k, v, 1, 1, 64, torch.float32)
        assert attention_close(out[:, :, :512], ref[:, :, :512]) and attention_close(out, ref), exact


def test_c5_real_routing_all_experts_k4096_narrow_output():
    """C5's routing (Zipf top-2 over 8 experts) on 4096 rows with K = 4096 and 256 output columns: 256-row tiles."""
    A, W, ex = inputs.moe_inputs(2048, 4096, 256, 8, 2, 4, torch.bfloat16)
    E = 8
    idx = torch.argsort(ex, stable=True).to(torch.int32)
    counts = torch.bincount(ex, minlength=E).to(torch.int32)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0)
    simlib.configure("lazy")
    out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, poison=9.0)
    assert rel_err(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2
