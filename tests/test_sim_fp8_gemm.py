"""Every fp8_gemm kernel path executed on the CPU in the host execution model (tests/sim: the kernel sources themselves,
compiled for the host) and compared with the oracle, with operands in guarded buffers and under the scheduling / DMA
landing variants.  The model sums each MFMA exactly, so where the output type rounds the same way the comparison is bit
for bit; the tolerance is the GPU tests' one.  What this adds to the GPU tests: it runs without a GPU, an access one byte
outside an operand stops the launch, and a transfer that is read before its wait (or a stage reused before its barrier)
gives a wrong answer in at least one variant instead of usually getting away with it."""
import pytest
import torch

from oracle import oracle as orc
from tests._util import rel_err
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn
FAST = ["lazy-reverse", "eager-interleaved"]
ALL = list(simlib.VARIANTS)


def _ops(m, n, k, seed, rowmajor):
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4)
    bt = (torch.randn(n, k, generator=g) * 0.5).to(E4)
    return a, (bt.t().contiguous() if rowmajor else bt.t())


# path (hx_fp8_gemm_path): 1 = 256x256 tiles, 2 = skinny (M <= 32), 3 = 256x256 guarded edges / K tail, 4 = row-major B
# read in place, 5 = 128-column tiles, 0 = plain kernel
@pytest.mark.parametrize("m,n,k,rowmajor,path", [
    (512, 512, 256, False, 5),      # (small problems prefer the 128-column tiles)
    (256, 256, 384, False, 5),
    (300, 260, 400, False, 3),      # ragged M, N and a 16-byte K tail
    (256, 256, 400, False, 3),
    (256, 512, 144, False, 3),      # one full k-tile + 16
    (256, 256, 16, False, 3),       # a single partial k-tile
    (256, 256, 256, True, 4),
    (300, 272, 400, True, 4),       # row-major B with ragged edges and a K tail
    (16, 512, 2048, False, 2),
    (32, 1024, 4096, False, 2),     # two 16-row blocks
    (8, 4096, 1024, False, 2),      # ticketed column groups (>= 12 per workgroup at this width)
    (1, 256, 512, False, 2),
    (16, 256, 16384, False, 2),     # K > 8192: A panel staged through the LDS
    (16, 256, 512, True, 0),        # row-major B for a skinny problem: transposed through the workspace (the query says 0)
    (40, 512, 1024, False, 5),      # 64-row decode tile
    (64, 1792, 1024, False, 5),
    (128, 1024, 2048, False, 5),
    (200, 640, 512, False, 5),
    (256, 256, 8192, False, 5),     # few tiles, long K: split-K slabs + reduce
    (33, 100, 1000, False, 0),      # K % 16 != 0: plain kernel
    (5, 7, 24, False, 0),
])
def test_paths_against_the_oracle(m, n, k, rowmajor, path):
    a, y = _ops(m, n, k, m + n + k, rowmajor)
    sa, sb = torch.tensor(1.5), torch.tensor(0.75)
    ref = orc.fp8_gemm(a, y, 1.5, 0.75, torch.bfloat16)
    for variant in FAST:
        simlib.configure(variant)
        out = simops.fp8_gemm(a, y, sa, sb, torch.bfloat16, want_path=path)
        assert rel_err(out, ref) <= 1e-2, variant


def test_path_1_the_256_tile_kernel_with_1_2_3_and_5_k_tiles():
    # enough tiles that the library picks 256x256 (the benchmark kernel); every k-tile count that has its own code shape:
    # 1 (prologue only), 2 (no steady-state iteration), 3 and 5 (steady state, odd counts end on either stage)
    for k in (128, 256, 384, 640):
        a, y = _ops(2048, 2304, k, k, False)
        ref = orc.fp8_gemm(a, y, 1.0, 1.0, torch.float32)
        simlib.configure("lazy-reverse")
        out = simops.fp8_gemm(a, y, None, None, torch.float32, want_path=1)
        assert rel_err(out, ref) <= 1e-6, k


@pytest.mark.parametrize("variant", ALL)
@pytest.mark.parametrize("m,n,k,rowmajor,path", [(300, 260, 400, False, 3), (256, 512, 384, True, 4),
                                                 (16, 1024, 2048, False, 2), (64, 896, 1024, False, 5)])
def test_every_variant_on_one_case_per_path(variant, m, n, k, rowmajor, path):
    a, y = _ops(m, n, k, 99, rowmajor)
    simlib.configure(variant)
    out = simops.fp8_gemm(a, y, None, None, torch.float16, want_path=path)
    assert rel_err(out, orc.fp8_gemm(a, y, 1.0, 1.0, torch.float16)) <= 1e-2


@pytest.mark.parametrize("end_flush", [True, False])
def test_ragged_shapes_touch_no_byte_outside_their_operands(end_flush):
    """Seeded sweep over ragged M / N / K (K % 16 == 0 and not), both layouts of B, every output type, with the operands'
    last (or first) byte against an inaccessible page."""
    import numpy as np
    rng = np.random.default_rng(3 if end_flush else 4)
    simlib.configure("lazy")
    for case in range(14):
        m = int(rng.choice([1, 7, 16, 17, 33, 100, 257, 300]))
        n = int(rng.choice([16, 24, 100, 128, 272, 520]))
        k = int(rng.choice([16, 48, 100, 128, 400, 1040]))
        rowmajor = bool(rng.integers(0, 2))
        od = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(0, 3))]
        a, y = _ops(m, n, k, 1000 + case, rowmajor)
        out = simops.fp8_gemm(a, y, None, None, od, end_flush=end_flush)
        assert rel_err(out, orc.fp8_gemm(a, y, 1.0, 1.0, od)) <= 1e-2, (case, m, n, k, rowmajor, od)


def test_ticket_word_with_stale_contents():
    """The ticketed decode kernel's workspace word needs no initialisation: run it with the word holding ones, a
    previous launch's tag and a large count."""
    a, y = _ops(16, 4096, 1024, 5, False)
    ref = orc.fp8_gemm(a, y, 1.0, 1.0, torch.bfloat16)
    simlib.configure("lazy")
    for stale in (0xFF, 0x00, 0x01, 0xA5):
        out = simops.fp8_gemm(a, y, None, None, torch.bfloat16, want_path=2, poison_ws=lambda nb: torch.full((nb,), stale, dtype=torch.uint8))
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), stale


def test_ticket_wait_gives_up_and_says_so():
    """A workgroup that draws a ticket before workgroup 0 has installed the launch's tag waits for the tag - for a bounded
    time.  With the workgroups run last to first, each to completion, the tag can never arrive: every workgroup but 0 must
    stop waiting, leave the give-up record in the second workspace word and end normally."""
    a, y = _ops(16, 4096, 1024, 5, False)
    ref = orc.fp8_gemm(a, y, 1.0, 1.0, torch.bfloat16)
    simlib.configure("lazy")
    zero = lambda nb: torch.zeros(nb, dtype=torch.uint8)  # (only the give-up record needs it: the ticket word itself may hold anything)
    with simlib.cus(8):
        after = []
        out = simops.fp8_gemm(a, y, None, None, torch.bfloat16, want_path=2, ws_after=after, ws_bytes=16, poison_ws=zero)   # in order: nothing to wait for
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
        words = after[0].view(torch.int64)
        assert int(words[0]) == 0 and int(words[1]) == 0     # ticket word cleared by the last draw, no give-up recorded
        with simlib.workgroups_last_to_first():
            after = []
            out = simops.fp8_gemm(a, y, None, None, torch.bfloat16, want_path=2, ws_after=after, ws_bytes=16, poison_ws=zero)  # completes: no hang, no fault
        words = after[0].view(torch.int64)
        assert int(words[1]) < 0                             # bit 63 set: somebody gave up
        # (here the result is complete all the same: workgroup 0, started last, draws every ticket the others left)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


# ---- opt-in path 6: row-major B streamed in place for a decode batch (HX_FEATURE_SKINNY_ROWMAJOR) ---------------------
@pytest.mark.parametrize("m,n,k,od", [
    (16, 256, 1024, torch.bfloat16),
    (1, 16, 1024, torch.float16),        # a single 16-byte chunk of columns
    (7, 144, 2048, torch.bfloat16),      # ragged last column group (one valid chunk), two k splits
    (16, 2048, 4096, torch.bfloat16),    # k split four ways (partial sums through the workspace)
    (32, 384, 8192, torch.bfloat16),     # two 16-row blocks, 64 slices per wave
    (20, 640, 1024, torch.float32),
])
def test_rowmajor_decode_kernel(m, n, k, od):
    from helion_amd import _lib
    g = torch.Generator().manual_seed(m + n + k)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4)
    y = (torch.randn(k, n, generator=g) * 0.5).to(E4)  # row-major [K, N]
    ref = orc.fp8_gemm(a, y, 1.5, 0.5, od)
    with simlib.features(_lib.HX_FEATURE_SKINNY_ROWMAJOR):
        for variant in ("lazy-reverse", "eager-interleaved"):
            simlib.configure(variant)
            out = simops.fp8_gemm(a, y, torch.tensor(1.5), torch.tensor(0.5), od, want_path=6, end_flush=(variant != "eager-interleaved"))
            assert rel_err(out, ref) <= 1e-2, variant
    # and switched off (the default) the same call takes the old route
    simlib.configure("lazy")
    out = simops.fp8_gemm(a, y, torch.tensor(1.5), torch.tensor(0.5), od, want_path=0 if m <= 16 else 4)
    assert rel_err(out, ref) <= 1e-2


@pytest.mark.parametrize("variant", ALL)
def test_rowmajor_decode_kernel_every_variant(variant):
    from helion_amd import _lib
    g = torch.Generator().manual_seed(8)
    a = (torch.randn(16, 2048, generator=g) * 0.5).to(E4)
    y = (torch.randn(2048, 1296, generator=g) * 0.5).to(E4)
    simlib.configure(variant)
    with simlib.features(_lib.HX_FEATURE_SKINNY_ROWMAJOR):
        out = simops.fp8_gemm(a, y, None, None, torch.bfloat16, want_path=6)
    assert rel_err(out, orc.fp8_gemm(a, y, 1.0, 1.0, torch.bfloat16)) <= 1e-2


def test_rowmajor_decode_kernel_ring_runs_on_across_column_groups():
    """More column groups than workgroups (a chip of 3 CUs in the model): a workgroup's ring carries the next group's first
    slices while the current group is reduced, and the last group re-fetches its own."""
    from helion_amd import _lib
    g = torch.Generator().manual_seed(9)
    a = (torch.randn(16, 1024, generator=g) * 0.5).to(E4)
    y = (torch.randn(1024, 1168, generator=g) * 0.5).to(E4)  # 10 column groups, the last with one valid chunk
    ref = orc.fp8_gemm(a, y, 1.0, 1.0, torch.bfloat16)
    with simlib.features(_lib.HX_FEATURE_SKINNY_ROWMAJOR), simlib.cus(3):
        for variant in ALL:
            simlib.configure(variant)
            out = simops.fp8_gemm(a, y, None, None, torch.bfloat16, want_path=6)
            assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), variant


def test_rowmajor_decode_needs_no_transpose_workspace_at_the_benchmark_shape():
    from helion_amd import _lib
    lib = simlib.load()
    assert lib.hx_fp8_gemm_workspace_bytes(16, 28672, 8192, 28672, 1) == 28672 * 8192  # default: transposed copy
    with simlib.features(_lib.HX_FEATURE_SKINNY_ROWMAJOR):
        assert lib.hx_fp8_gemm_workspace_bytes(16, 28672, 8192, 28672, 1) == 0
        assert lib.hx_fp8_gemm_path(16, 28672, 8192, 8192, 28672, 1, 28672, 1 << 20, 1 << 20, 1 << 20) == 6


# ---- opt-in: any K through the MFMA kernels (HX_FEATURE_FP8_GEMM_ANY_K) --------------------------------------------------
@pytest.mark.parametrize("m,n,k,rowmajor", [
    (300, 260, 1000, False),   # K % 16 = 8: both operands padded, guarded-edge tile kernel
    (33, 100, 1001, False),    # odd K: byte-aligned rows
    (16, 512, 2047, False),    # a decode batch: K padded to 2048, the skinny kernel
    (64, 1792, 1023, False),   # 64-row decode tile
    (200, 272, 100, True),     # row-major B: transposed and padded in one pass
    (5, 7, 24, False),         # K % 16 = 8, tiny
    (256, 256, 3, True),       # K below one chunk
])
def test_any_k_through_the_mfma_kernels(m, n, k, rowmajor):
    import ctypes
    from helion_amd import _lib
    a, y = _ops(m, n, k, 77 + k, rowmajor)
    ref = orc.fp8_gemm(a, y, 1.5, 0.75, torch.bfloat16)
    lib, c = simlib.load(), (ctypes.c_uint64 * 4)()
    for variant in FAST:
        simlib.configure(variant)
        lib.hx_sim_counters(c)
        before = c[0]
        with simlib.features(_lib.HX_FEATURE_FP8_GEMM_ANY_K):
            out = simops.fp8_gemm(a, y, torch.tensor(1.5), torch.tensor(0.75), torch.bfloat16, want_path=0)
        lib.hx_sim_counters(c)
        assert c[0] > before, "the plain kernel ran (it has no cross-lane instructions): the repacked route was not taken"
        assert rel_err(out, ref) <= 1e-2, variant


def test_any_k_route_really_runs_matrix_instructions():
    """The repacked call must multiply with MFMAs (the model counts cross-lane instructions; the plain kernel has none)."""
    import ctypes
    from helion_amd import _lib
    lib = simlib.load()
    a, y = _ops(64, 128, 1000, 3, False)
    simlib.configure("lazy")

    def cross_lane_instructions(mask):
        c = (ctypes.c_uint64 * 4)()
        lib.hx_sim_counters(c)
        before = c[0]
        with simlib.features(mask):
            simops.fp8_gemm(a, y, None, None, torch.bfloat16)
        lib.hx_sim_counters(c)
        return c[0] - before

    assert cross_lane_instructions(0) == 0
    assert cross_lane_instructions(_lib.HX_FEATURE_FP8_GEMM_ANY_K) > 100


# ---- opt-in: the persistent 256x256 kernel (HX_FEATURE_FP8_GEMM_PERSISTENT) ------------------------------------------------
def _persistent(m, n, k, cus, variant, od=torch.bfloat16, seed=5):
    from helion_amd import _lib
    a, y = _ops(m, n, k, seed + m + n + k, False)
    simlib.configure(variant)
    with simlib.features(_lib.HX_FEATURE_FP8_GEMM_PERSISTENT), simlib.cus(cus):
        simlib.work()
        out = simops.fp8_gemm(a, y, torch.tensor(1.25), torch.tensor(0.5), od, want_path=7)
        w = simlib.work()
    return out, orc.fp8_gemm(a, y, 1.25, 0.5, od), w


@pytest.mark.parametrize("variant", ALL)
def test_persistent_kernel_every_variant(variant):
    """16 tiles on 8 workgroups: every workgroup hands one tile's accumulators over inside the next tile's first k-tile and
    ends with the plain epilogue.  K = 512 is the shortest the path takes (k-tiles 0, 1, nk-2, nk-1 and no steady loop)."""
    out, ref, w = _persistent(1024, 1024, 512, 8, variant)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    assert w["workgroups"] == 8 and w["mfma"] == 16 * 4 * 4 * 64  # 16 tiles x 4 k-tiles x 4 waves x 64 MFMAs: the hand-over adds none


@pytest.mark.parametrize("m,n,k,cus,variant,od", [
    (1024, 1280, 768, 8, "lazy", torch.bfloat16),            # 20 tiles on 8 workgroups: 3 / 2 tiles per workgroup; a steady loop of one k-tile
    (2048, 1024, 1024, 16, "lazy-reverse", torch.bfloat16),  # 32 tiles on 16 workgroups
    (1024, 1024, 1280, 8, "eager-interleaved", torch.float16),
])
def test_persistent_kernel_shapes(m, n, k, cus, variant, od):
    out, ref, _ = _persistent(m, n, k, cus, variant, od)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_persistent_kernel_is_chosen_only_where_every_workgroup_gets_two_tiles():
    from helion_amd import _lib
    lib = simlib.load()
    with simlib.features(_lib.HX_FEATURE_FP8_GEMM_PERSISTENT), simlib.cus(8):
        def path(m, n, k):
            return lib.hx_fp8_gemm_path(m, n, k, k, 1, k, n, None, None, None)
        assert path(1024, 1024, 512) == 7
        assert path(768, 768, 512) != 7       # 9 tiles on 8 workgroups
        assert path(1024, 1024, 256) != 7     # a single k-tile pair: nothing to overlap the epilogue with
        assert path(1024, 1024, 640) != 7     # K % 256 != 0
    with simlib.cus(8):
        assert lib.hx_fp8_gemm_path(1024, 1024, 512, 512, 1, 512, 1024, None, None, None) != 7  # off by default


# ---- opt-in: decode batches of 33..256 rows with separate A / B rings (HX_FEATURE_FP8_GEMM_DECODE_RING) ---------------------
def _decode_ring(m, n, k, variant, od=torch.bfloat16, **kw):
    from helion_amd import _lib
    a, y = _ops(m, n, k, 11 + m + n + k, False)
    sa, sb = torch.tensor(1.25), torch.tensor(0.5)
    simlib.configure(variant)
    base = simops.fp8_gemm(a, y, sa, sb, od, want_path=5)
    with simlib.features(_lib.HX_FEATURE_FP8_GEMM_DECODE_RING):
        simlib.work()
        out = simops.fp8_gemm(a, y, sa, sb, od, want_path=8, **kw)
        w = simlib.work()
    return out, base, orc.fp8_gemm(a, y, 1.25, 0.5, od), w


@pytest.mark.parametrize("variant", ALL)
# 64: B waves issue pairs of k-tiles into a ring of 8; 128 / 192 / 256: single k-tiles into a ring of 7 / 5 / 4 (192: a tile only this kernel has)
@pytest.mark.parametrize("m", [64, 128, 192, 256])
def test_decode_ring_kernel_every_variant(variant, m):
    out, base, ref, _ = _decode_ring(m, 256, 2560, variant)   # 20 k-tiles: every ring wraps at least twice
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))  # same MFMA order as the kernel it replaces
    assert rel_err(out, ref) <= 1e-2


@pytest.mark.parametrize("m,n,k,od", [
    (33, 100, 128, torch.bfloat16),     # a single k-tile: the prologue re-fetches it into every stage
    (40, 512, 1024, torch.bfloat16),    # few tiles, K >= 1024: split-K slabs + reduce
    (100, 640, 512, torch.float16),     # ragged rows and a column pitch below 128
    (64, 144, 256, torch.float32),      # two k-tiles, a last tile of 16 columns
    (65, 112, 1280, torch.bfloat16),
    (128, 1792, 1024, torch.bfloat16),
    (96, 128, 8192, torch.bfloat16),    # 64 k-tiles in 8 splits
    (130, 256, 1024, torch.bfloat16),   # 192-row tile, 62 rows of padding
    (160, 144, 128, torch.float16),     # 192-row tile, a single k-tile
    (200, 640, 512, torch.bfloat16),    # 256-row tile
    (256, 384, 2048, torch.float32),
])
def test_decode_ring_kernel_shapes(m, n, k, od):
    for variant in FAST:
        out, base, ref, _ = _decode_ring(m, n, k, variant, od)
        assert torch.equal(out.view(torch.uint8), base.view(torch.uint8)), variant
        assert rel_err(out, ref) <= 1e-2, variant


def test_decode_ring_kernel_keeps_twice_the_weight_bytes_in_flight():
    """What the kernel is for: with 128 rows the single-ring kernel lets 2 - 3 weight stages (32 - 48 KB) per workgroup be in
    flight, the two-ring one 5 - 6 (80 - 96 KB).  Counted by the model under lazy landing: bytes of B issued and not yet
    covered by a wait of the issuing wave, at their peak and right after the waits."""
    from helion_amd import _lib
    a, y = _ops(128, 896, 2048, 3, False)
    simlib.configure("lazy")
    fig = {}
    for mask, path in ((0, 5), (_lib.HX_FEATURE_FP8_GEMM_DECODE_RING, 8)):
        with simlib.features(mask):
            simlib.work()
            simops.fp8_gemm(a, y, None, None, torch.bfloat16, want_path=path, ws_bytes=0, in_flight_of_b=True)  # (no workspace: no split-K)
            fig[path] = simlib.work()
    assert fig[5]["dma_in_flight_max"] <= 3 * 16384 + 4096 and fig[8]["dma_in_flight_max"] >= 6 * 16384
    assert fig[8]["dma_in_flight_after_waits"] >= 2 * fig[5]["dma_in_flight_after_waits"]
