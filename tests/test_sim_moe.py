"""The grouped-GEMM kernels, the routing-table kernels, the top-k entry and the entry point that allocates nothing,
executed on the CPU in the host execution model (tests/sim) against the oracle: every kernel path, ragged column tiles,
partial last k-tiles, 4-byte-aligned rows, empty experts, uncovered rows, more experts than one table chunk holds."""
import pytest
import torch

from helion_amd import inputs
from oracle import oracle as orc
from tests._util import rel_err
from tests.sim import simlib, simops


def _tables(ex, E):
    idx = torch.argsort(ex, stable=True).to(torch.int32)
    counts = torch.bincount(ex, minlength=E).to(torch.int32)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0)
    return counts, offsets, idx


# path (hx_moe_path): 0 fp32-FMA kernel, 1 / 2 / 3 MFMA with 32- / 128- / 256-row tiles, 4 = 128-row tiles with a partial
# last k-tile, 5 = the same with A fetched in 4-byte pieces
CASES = [
    (1000, 500, 200, 30, 1, torch.float16, 5),   # the reference's own check shape (examples/moe_matmul_ogs.py:186)
    (1000, 504, 200, 30, 1, torch.float16, 4),
    (333, 2, 8, 3, 1, torch.bfloat16, 5),
    (40, 126, 64, 4, 1, torch.bfloat16, 5),
    (37, 101, 24, 3, 1, torch.bfloat16, 0),      # odd K
    (37, 100, 19, 3, 1, torch.bfloat16, 0),      # N % 8 != 0
    (512, 256, 512, 4, 1, torch.bfloat16, 2),
    (700, 128, 256, 5, 1, torch.float16, 2),
    (300, 64, 256, 16, 1, torch.bfloat16, 2),    # most tiles nearly empty
    (512, 128, 384, 4, 1, torch.bfloat16, 2),    # ragged last column tile
    (256, 64, 8, 2, 1, torch.bfloat16, 2),       # one valid 16-byte chunk of columns
    (300, 192, 200, 5, 1, torch.bfloat16, 2),
    (32, 256, 512, 8, 1, torch.bfloat16, 1),     # a decode batch: 32-row tiles
    (16, 512, 264, 4, 2, torch.float16, 1),
    (7, 64, 128, 3, 1, torch.bfloat16, 1),
    (24, 128, 136, 40, 1, torch.bfloat16, 1),    # more experts than rows
    (300, 8, 64, 3, 1, torch.bfloat16, 4),       # the only k-tile is partial, a single chunk
    (300, 72, 136, 3, 1, torch.float16, 4),
    (20, 200, 264, 4, 1, torch.bfloat16, 4),
    (3000, 64, 64, 700, 1, torch.bfloat16, 2),   # tile table built 256 experts at a time (three chunks, many empty)
    (6144, 128, 2048, 2, 1, torch.bfloat16, 3),  # 256-row tiles
]


@pytest.mark.parametrize("T,K,N,E,topk,dtype,path", CASES)
def test_paths_against_the_oracle(T, K, N, E, topk, dtype, path):
    A, W, ex = inputs.moe_inputs(T // topk, K, N, E, topk, seed=T + K, dtype=dtype)
    ref = orc.moe_matmul_ogs_reference(A, W, ex)
    counts, offsets, idx = _tables(ex, E)
    for variant in (["lazy-reverse"] if path == 3 else ["lazy-reverse", "eager-interleaved"]):
        simlib.configure(variant)
        out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=path, poison=7.0)
        assert rel_err(out, ref) <= 1e-2, variant


@pytest.mark.parametrize("variant", list(simlib.VARIANTS))
@pytest.mark.parametrize("T,K,N,E,dtype,path", [(600, 192, 264, 3, torch.bfloat16, 2), (30, 128, 256, 5, torch.float16, 1),
                                                (500, 120, 200, 4, torch.bfloat16, 4), (500, 70, 200, 4, torch.float16, 5)])
def test_every_variant_on_one_case_per_mfma_kernel(variant, T, K, N, E, dtype, path):
    A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=3, dtype=dtype)
    counts, offsets, idx = _tables(ex, E)
    simlib.configure(variant)
    out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=path)
    assert rel_err(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2


@pytest.mark.parametrize("K,N", [(128, 256), (96, 40)])
def test_empty_experts_and_uncovered_rows_are_zero(K, N):
    A, W, ex = inputs.moe_inputs(400, K, N, 6, 1, seed=1, dtype=torch.bfloat16)
    ex[ex == 2] = 4
    counts, offsets, idx = _tables(ex, 6)
    counts[1] = 0  # expert 1 switched off: its rows are covered by nobody
    simlib.configure("lazy")
    out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, poison=3.0)
    ref = orc.moe_matmul_ogs(A, W, counts, offsets, idx)
    assert rel_err(out, ref) <= 1e-2
    assert bool((out[ex == 1] == 0).all())


def test_static_entry_equals_the_workspace_one_bit_for_bit_second_call_smaller():
    simlib.configure("lazy")
    for T, K, N, E, dtype, path in [(6000, 128, 256, 8, torch.bfloat16, 2), (700, 128, 264, 5, torch.float16, 2),
                                    (1000, 500, 200, 30, torch.float16, 5), (900, 251, 200, 6, torch.float16, 0)]:
        A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=T, dtype=dtype)
        if E > 2:
            ex[ex == 1] = 0
        counts, offsets, idx = _tables(ex, E)
        counts[E - 1] = 0
        a = simops.moe_grouped_gemm(A, W, counts, offsets, idx, static=False, want_path=path, poison=2.0)
        b = simops.moe_grouped_gemm(A, W, counts, offsets, idx, static=True, poison=-1.0)
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
        assert bool((b[ex == E - 1] == 0).all()) and bool(b.float().abs().max() > 0)


@pytest.mark.parametrize("T,E,dtype", [(1, 4, torch.int64), (1000, 8, torch.int64), (5000, 300, torch.int32), (40000, 8, torch.int64),
                                       (70000, 64, torch.int32), (3000, 512, torch.int64)])
def test_routing_tables(T, E, dtype):
    g = torch.Generator().manual_seed(T)
    ids = torch.randint(0, E, (T,), generator=g).to(dtype)
    for variant in ("lazy", "eager-interleaved"):
        simlib.configure(variant)
        counts, offsets, idx, mx = simops.moe_routing(ids, E)
        rc = torch.bincount(ids.long(), minlength=E).int()
        assert torch.equal(counts, rc) and torch.equal(idx, torch.argsort(ids.long(), stable=True).int())
        assert int(offsets[0]) == 0 and torch.equal(offsets[1:], torch.cumsum(rc, 0).int()) and int(mx) == int(rc.max())


@pytest.mark.parametrize("T,E,dtype", [(3000, 513, torch.int64), (5000, 1100, torch.int32), (20000, 2048, torch.int64), (70000, 2048, torch.int32),
                                       (40000, 1500, torch.int64), (100, 2000, torch.int32)])
def test_routing_tables_for_513_to_2048_experts(T, E, dtype):
    """Opt-in (HX_FEATURE_ROUTING_WIDE): the same kernels with LDS tables for 2048 experts, two experts per work-item in the
    scans; one workgroup up to 32768 rows, count / scan / scatter launches above."""
    from helion_amd import _lib
    g = torch.Generator().manual_seed(T + E)
    ids = torch.randint(0, E, (T,), generator=g).to(dtype)
    ids[::7] = E - 1   # a crowded last expert, and most experts nearly empty at the small T
    lib = simlib.load()
    simlib.configure("lazy")
    out = [torch.zeros(n, dtype=torch.int32) for n in (E, E + 1, max(T, 1), 1)]
    assert lib.hx_moe_routing(ids.data_ptr(), int(dtype == torch.int64), T, E, *[t.data_ptr() for t in out], None, 0, None) != 0  # off by default
    lib.hx_sim_reset()
    with simlib.features(_lib.HX_FEATURE_ROUTING_WIDE):
        for variant in ("lazy", "eager-interleaved"):
            simlib.configure(variant)
            counts, offsets, idx, mx = simops.moe_routing(ids, E)
            rc = torch.bincount(ids.long(), minlength=E).int()
            assert torch.equal(counts, rc) and torch.equal(idx, torch.argsort(ids.long(), stable=True).int())
            assert int(offsets[0]) == 0 and torch.equal(offsets[1:], torch.cumsum(rc, 0).int()) and int(mx) == int(rc.max())
        assert lib.hx_moe_routing(ids.data_ptr(), int(dtype == torch.int64), T, 2049, *[t.data_ptr() for t in out], None, 0, None) != 0


def test_routing_skips_ids_out_of_range():
    ids = torch.tensor([3, -1, 0, 9, 3, 2, 100, 0], dtype=torch.int64)
    simlib.configure("lazy")
    counts, offsets, idx, mx = simops.moe_routing(ids, 4)
    assert counts.tolist() == [2, 0, 1, 2] and offsets.tolist() == [0, 2, 2, 3, 5] and idx.tolist() == [2, 7, 5, 0, 4, -1, -1, -1]


@pytest.mark.parametrize("tokens,K,N,E,topk,dtype", [(300, 128, 256, 6, 2, torch.bfloat16), (50, 100, 264, 3, 2, torch.float16),
                                                     (9, 64, 128, 8, 4, torch.bfloat16)])
def test_topk_entry_equals_the_replicated_rows_form(tokens, K, N, E, topk, dtype):
    A, W, ex = inputs.moe_inputs(tokens, K, N, E, topk, seed=tokens, dtype=dtype)
    simlib.configure("lazy-reverse")
    out = simops.moe_topk(A[::topk].contiguous(), W, ex, topk)
    assert rel_err(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2


# ---- opt-in: the 256-row tiles in persistent workgroups (HX_FEATURE_MOE_PERSISTENT, hx_moe_path 6) ---------------------------
def _persistent(T, K, N, E, cus, variant, dtype=torch.bfloat16, drop_expert=None, with_base=True):
    from helion_amd import _lib
    A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=T + K, dtype=dtype)
    counts, offsets, idx = _tables(ex, E)
    if drop_expert is not None:
        counts[drop_expert] = 0   # its rows are covered by nobody: they must come out zero
    simlib.configure(variant)
    with simlib.cus(cus):
        base = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=3, poison=7.0) if with_base else None
        with simlib.features(_lib.HX_FEATURE_MOE_PERSISTENT):
            simlib.work()
            out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=6, poison=5.0)
            w = simlib.work()
    w["row_tiles"] = int(((counts + 255) // 256).sum())
    return out, base, orc.moe_matmul_ogs(A, W, counts, offsets, idx), w


@pytest.mark.parametrize("T,K,N,E,cus,variant,dtype,with_base", [
    (6144, 256, 2048, 2, 8, "lazy", torch.bfloat16, True),                # the shortest K the path takes: k-tiles 0, 1, nk-2, nk-1 only
    (6144, 256, 2048, 3, 16, "lazy-reverse", torch.bfloat16, False),      # 200-odd tiles on 16 workgroups: a ragged last step
    (6144, 384, 2048, 3, 8, "eager-interleaved", torch.float16, False),   # six k-tiles: a steady loop of two
] + ([(6400, 512, 2048, 4, 24, "lazy-interleaved", torch.bfloat16, True)] if __import__("os").environ.get("HX_SIM_SWEEP") == "1" else []))
def test_persistent_grouped_kernel(T, K, N, E, cus, variant, dtype, with_base):
    """Every workgroup hands each tile's accumulators over inside the next tile's first k-tile and ends with a plain
    epilogue; rows that are not stored go to the sink behind the row flags.  Bit-equal to the kernel it replaces."""
    out, base, ref, w = _persistent(T, K, N, E, cus, variant, dtype, with_base=with_base)
    if with_base:
        assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    assert rel_err(out, ref) <= 1e-2
    # 4 waves x 128 MFMAs per tile and k-tile: the hand-over adds none
    assert w["mfma"] == w["row_tiles"] * (N // 256) * (K // 64) * 512


def test_persistent_grouped_kernel_with_an_expert_switched_off():
    out, _, ref, _ = _persistent(6144, 256, 2048, 3, 8, "lazy", drop_expert=1, with_base=False)
    assert rel_err(out, ref) <= 1e-2 and bool((ref == 0).any())


def test_persistent_grouped_kernel_is_chosen_only_for_whole_column_tiles_and_even_k_tiles():
    from helion_amd import _lib
    lib = simlib.load()
    with simlib.cus(8):
        def path(T, K, N, E):
            return lib.hx_moe_path(T, K, N, E, 1, None, None, None)
        assert path(6144, 256, 2048, 2) == 3                  # off by default
        with simlib.features(_lib.HX_FEATURE_MOE_PERSISTENT):
            assert path(6144, 256, 2048, 2) == 6
            assert path(6144, 128, 2048, 2) == 3              # two k-tiles: nothing to overlap with
            assert path(6144, 320, 2048, 2) != 6              # an odd number of k-tiles
            assert path(6144, 256, 2176, 2) == 3              # a ragged last column tile
            assert path(1024, 256, 2048, 8) == 2              # small experts keep the 128-row tiles
            assert lib.hx_moe_workspace_bytes(6144, 2) >= 1024 + 6144


def test_persistent_grouped_kernel_through_the_top_k_entry():
    """a_div = 2: C row r is the product of A row r / 2; routing on the device, the sink inside the top-k workspace."""
    from helion_amd import _lib
    A, W, ex = inputs.moe_inputs(3072, 256, 2048, 2, 2, seed=9, dtype=torch.bfloat16)
    simlib.configure("lazy-reverse")
    with simlib.cus(8), simlib.features(_lib.HX_FEATURE_MOE_PERSISTENT):
        assert simlib.load().hx_moe_path(6144, 256, 2048, 2, 2, None, None, None) == 6
        out = simops.moe_topk(A[::2].contiguous(), W, ex, 2)
    assert rel_err(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2


# ---- opt-in: odd K / N % 8 != 0 through the MFMA kernels (HX_FEATURE_MOE_ANY_SHAPE) -----------------------------------------
@pytest.mark.parametrize("T,K,N,E,dtype", [
    (37, 101, 24, 3, torch.bfloat16),      # odd K: A and W repacked, C written in place
    (37, 100, 19, 3, torch.bfloat16),      # N % 8 != 0: W and C padded, C cropped back
    (300, 251, 203, 5, torch.float16),     # both
    (600, 65, 260, 4, torch.bfloat16),     # K8 = 72: a partial last k-tile after padding
    (20, 1, 9, 2, torch.bfloat16),         # a single k, a single padded chunk of columns
])
def test_any_shape_through_the_mfma_kernels(T, K, N, E, dtype):
    import ctypes
    from helion_amd import _lib
    A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=T + K + N, dtype=dtype)
    counts, offsets, idx = _tables(ex, E)
    counts[E - 1] = 0   # an expert switched off: its rows must come out zero after the crop as well
    ref = orc.moe_matmul_ogs(A, W, counts, offsets, idx)
    lib, c = simlib.load(), (ctypes.c_uint64 * 4)()
    assert lib.hx_moe_workspace_bytes_shape(T, K, N, E) == lib.hx_moe_workspace_bytes(T, E)   # off by default
    for variant in ("lazy-reverse", "eager-interleaved"):
        simlib.configure(variant)
        with simlib.features(_lib.HX_FEATURE_MOE_ANY_SHAPE):
            assert lib.hx_moe_workspace_bytes_shape(T, K, N, E) > lib.hx_moe_workspace_bytes(T, E)
            lib.hx_sim_counters(c)
            before = c[0]
            out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=0, poison=4.0)
            lib.hx_sim_counters(c)
        assert c[0] > before, "no cross-lane instruction ran: the fp32 kernel took the call, not the repacked route"
        assert rel_err(out, ref) <= 1e-2, variant
        assert bool((out[ex == E - 1] == 0).all())
