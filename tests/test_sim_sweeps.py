"""Address-extent sweeps in the host execution model (tests/sim): the kernels whose global->LDS DMA addresses are
computed by hand (clamped rows, re-read chunks, partial last tiles) are run over every residue class of the ragged
dimension with each operand's last byte against an inaccessible page, so a clamp that is off by one row or chunk stops
the launch with the address, and the results are still compared with the oracle.  The default run covers every residue
once at small sizes; HX_SIM_SWEEP=1 widens it (sequence lengths up to 4200, all K tails at several tile counts)."""
import os

import pytest
import torch

from helion_amd import inputs
from oracle import oracle as orc
from tests._util import attention_close, rel_err
from tests.sim import simlib, simops

E4 = torch.float8_e4m3fn
WIDE = os.environ.get("HX_SIM_SWEEP", "0") not in ("", "0")


def _att(s, d, exact, layout, seed=0, flush=True):
    g = torch.Generator().manual_seed(seed + s)
    q, k = (torch.randn(1, s, d, generator=g).to(E4) for _ in range(2))
    v = torch.randn(1, d, s, generator=g).to(E4)
    out = simops.fp8_attention(q, k, v, 1, 1, torch.float32, exact, layout, end_flush=flush, want_path=1)
    ref = orc.fp8_attention(q, k, v, 1, 1, torch.float32) if exact else orc.fp8_attention_tiled(q, k, v, 1, 1, 64, torch.float32)
    assert attention_close(out, ref), (s, d, exact, layout, rel_err(out, ref))


def test_attention_every_sequence_length_residue_strided_v():
    """[S][D] layout of V (any S): every S from 1 to 200 (each residue mod 64 at 1, 2, 3 and 4 tiles), alternating modes
    and head dims; the wide run goes on to 4200 in steps that visit every residue mod 64 at every tile-count parity."""
    simlib.configure("lazy")
    lens = list(range(1, 201)) + ([576 + 7 * i for i in range(64)] + [1100 + 67 * i for i in range(40)] + [4097, 4200] if WIDE else [])
    for i, s in enumerate(lens):
        _att(s, 64 if i % 2 else 128, bool((i // 2) % 2), "SD")


def test_attention_every_multiple_of_16_contiguous_v():
    """[D][S] layout of V (S % 16 == 0): every multiple of 16 up to 704 (11 tiles: the first steady-state rounds of pass
    1), both modes; the wide run adds lengths up to 4160."""
    simlib.configure("lazy-reverse")
    lens = list(range(16, 720, 16)) + ([1024 + 48 * i for i in range(24)] + [4096, 4160] if WIDE else [])
    for i, s in enumerate(lens):
        _att(s, 128 if i % 3 else 64, bool(i % 2), "DS", flush=bool(i % 5))


def _gemm(m, n, k, rowmajor, od=torch.bfloat16, flush=True):
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4)
    bt = (torch.randn(n, k, generator=g) * 0.5).to(E4)
    y = bt.t().contiguous() if rowmajor else bt.t()
    out = simops.fp8_gemm(a, y, None, None, od, end_flush=flush)
    assert rel_err(out, orc.fp8_gemm(a, y, 1.0, 1.0, od)) <= 1e-2, (m, n, k, rowmajor)


def test_fp8_gemm_every_k_tail_and_ragged_edges():
    """Guarded-edge instantiations of the 256x256 tile kernel (both layouts of B) and the 128-column tiles: every K tail
    (K % 128 = 16 .. 112) at one and at three k-tiles, with M and N one below / one above / well off a tile edge."""
    simlib.configure("lazy")
    ks = [16 * t for t in range(1, 9)] + [256 + 16 * t for t in range(1, 8)]
    shapes = [(257, 272), (255, 240), (300, 16), (17, 528)]
    if WIDE:
        ks += [512 + 16 * t for t in range(0, 8)] + [1024 + 48]
        shapes += [(512, 512), (511, 496), (33, 1040), (1000, 48)]
    for i, k in enumerate(ks):
        m, n = shapes[i % len(shapes)]
        _gemm(m, n, k, rowmajor=False, flush=bool(i % 2))
        _gemm(m, n, k, rowmajor=True, flush=not bool(i % 2))


def test_grouped_gemm_every_k_tail():
    """128-row tiles with a partial last k-tile: every K % 64 in steps of 8 (16-byte rows) and of 2 (4-byte rows)."""
    simlib.configure("lazy")
    ks = list(range(8, 136, 8)) + list(range(2, 72, 6)) + [126, 130, 190]
    if WIDE:
        ks = list(range(2, 260, 2))
    for i, k in enumerate(ks):
        T, N, E = (150, 136, 3) if i % 2 else (70, 264, 5)
        A, W, ex = inputs.moe_inputs(T, k, N, E, 1, seed=k, dtype=torch.bfloat16 if i % 3 else torch.float16)
        idx = torch.argsort(ex, stable=True).to(torch.int32)
        counts = torch.bincount(ex, minlength=E).to(torch.int32)
        offsets = torch.zeros(E + 1, dtype=torch.int32)
        offsets[1:] = torch.cumsum(counts, 0)
        out = simops.moe_grouped_gemm(A, W, counts, offsets, idx, end_flush=bool(i % 2))
        assert rel_err(out, orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2, k
