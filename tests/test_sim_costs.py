"""The per-tile work of the three hot kernels, counted by the host execution model (tests/sim) while it executes them:
wave-level MFMA instructions, bytes moved global -> LDS by DMA, LDS bytes the kernels read and write themselves, barriers.
These are the figures the design's budget arguments rest on (LDS bytes per MFMA cycle, DMA bytes per k-tile, the exact
attention mode executing 1.5 times the counted flops); here they are measured on the kernel source instead of asserted
in prose.  No timing is involved."""
import torch

from helion_amd import inputs
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn
KB = 1024


def _fp8_gemm_work(k):
    g = torch.Generator().manual_seed(0)
    a = (torch.randn(2048, k, generator=g) * 0.5).to(E4)
    bt = (torch.randn(2304, k, generator=g) * 0.5).to(E4)
    simlib.configure("eager")
    simlib.work()
    simops.fp8_gemm(a, bt.t(), None, None, torch.bfloat16, want_path=1)
    return simlib.work()


def test_fp8_gemm_256_tile_kernel_per_k_tile():
    """hx_fp8_gemm_tile256 (the benchmark kernel): per workgroup and 128-deep k-tile 256 MFMAs of 16x16x128 (64 per wave =
    2048 matrix-pipe cycles per SIMD), 64 KB fetched by DMA (A 32 KB + B 32 KB, each byte once), 128 KB of fragment reads
    (every A and every B fragment is read by two waves) and two barriers; outside the k loop one set of fragments (128 KB)
    and the output staged once through the LDS (128 KB written, 128 KB read for a 16-bit output)."""
    w3, w5 = _fp8_gemm_work(384), _fp8_gemm_work(640)
    wgs = w3["workgroups"]
    assert wgs == (2048 // 256) * (2304 // 256) == w5["workgroups"]
    per = {k: (w5[k] - w3[k]) / (2 * wgs) for k in w3}
    assert per["mfma"] == 256 and per["dma_bytes"] == 64 * KB and per["lds_read"] == 128 * KB and per["lds_write"] == 0
    assert per["barriers"] == 2
    fixed = {k: w3[k] / wgs - 3 * per[k] for k in w3}
    assert fixed["mfma"] == 0 and fixed["dma_bytes"] == 0  # nothing is fetched twice, nothing multiplied outside the loop
    assert fixed["lds_read"] == 256 * KB and fixed["lds_write"] == 128 * KB
    # LDS traffic per k-tile against the matrix pipe: (128 KB read + 64 KB written by DMA) / 128 B per clock = 1536 of
    # the 2048 cycles the MFMAs take: the budget the design quotes
    assert (per["lds_read"] + per["dma_bytes"]) / 128 == 1536


def _att_work(s, exact):
    g = torch.Generator().manual_seed(0)
    q, k = (torch.randn(1, s, 128, generator=g).to(E4) for _ in range(2))
    v = torch.randn(1, 128, s, generator=g).to(E4)
    simlib.configure("eager")
    simlib.work()
    simops.fp8_attention(q, k, v, 1, 1, torch.float32, exact, "DS", want_path=1)
    return simlib.work()


def test_fp8_attention_per_key_tile():
    """hx_fp8_attention_pipe at D = 128, per workgroup (128 queries) and 64-key tile: the online mode issues 32 MFMAs of
    32x32x64 (16 for S = Q K^T, 16 for P V: the counted flops), the exact-max mode 48 (its first pass multiplies Q K^T
    once more: 1.5 times the counted work); K and V are each fetched once per pass that uses them (16 KB online, 24 KB
    exact, plus the re-fetches that keep the DMA count constant past the last tile)."""
    for exact, mfma, dma in ((False, 32, 16 * KB), (True, 48, 24 * KB)):
        a, b = _att_work(1024, exact), _att_work(2048, exact)
        for w, s in ((a, 1024), (b, 2048)):
            n = (s // 128) * (s // 64)
            assert w["mfma"] == mfma * n, (exact, s)
        # bytes per (workgroup, tile) from the difference of the two lengths: the fixed re-fetches cancel
        na, nb = (1024 // 128) * (1024 // 64), (2048 // 128) * (2048 // 64)
        tail_a, tail_b = a["dma_bytes"] - dma * na, b["dma_bytes"] - dma * nb
        assert tail_a >= 0 and tail_b >= 0
        assert tail_a / (1024 // 128) == tail_b / (2048 // 128)  # the same few extra tiles per workgroup at either length
        assert tail_a / (1024 // 128) <= 8 * 8 * KB


def test_grouped_gemm_256_tile_kernel_per_k_tile():
    """hx_gemm16_tile256 (the grouped GEMM's kernel at the benchmark shape): per workgroup and 64-deep k-tile 512 MFMAs
    of 16x16x32 (128 per wave = 2048 matrix-pipe cycles per SIMD, as in the fp8 kernel), 64 KB by DMA (256 gathered rows
    of A and 256 columns of W, 32 KB each), 128 KB of fragment reads, two barriers: the same LDS budget as the fp8 kernel's."""
    def run(K):
        A, W, ex = inputs.moe_inputs(6144, K, 2048, 2, 1, seed=1, dtype=torch.bfloat16)
        idx = torch.argsort(ex, stable=True).to(torch.int32)
        counts = torch.bincount(ex, minlength=2).to(torch.int32)
        offsets = torch.zeros(3, dtype=torch.int32)
        offsets[1:] = torch.cumsum(counts, 0)
        simlib.configure("eager")
        simops.moe_grouped_gemm(A[:1], W[:, :, :8], torch.tensor([1, 0]), torch.tensor([0, 1, 1]), torch.tensor([0]))  # (warm)
        simlib.work()
        simops.moe_grouped_gemm(A, W, counts, offsets, idx, want_path=3)
        return simlib.work(), int(((counts + 255) // 256).sum()) * (2048 // 256)

    (w2, tiles), (w4, tiles4) = run(128), run(256)
    assert tiles == tiles4
    per = {k: (w4[k] - w2[k]) / (2 * tiles) for k in w2}
    assert per["mfma"] == 512 and per["dma_bytes"] == 64 * KB and per["lds_read"] == 128 * KB
    assert per["barriers"] == 2
