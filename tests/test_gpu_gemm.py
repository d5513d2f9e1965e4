"""GPU parity of hx_fp8_gemm (all three kernels) against the CPU oracle, the golden fixture and, at the
benchmark sizes, sampled rows plus a checksum identity.  Everything goes through the C ABI."""
import ctypes
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
E4M3 = torch.float8_e4m3fn
G = pathlib.Path(__file__).resolve().parent / "golden"


def _path(m, n, k):
    return _lib.load().hx_fp8_gemm_path(m, n, k, k, 1, k, n, 1 << 20, 1 << 20, 1 << 20)


@pytest.mark.parametrize("m,n,k,path", [
    (4096, 4096, 128, 1), (2048, 6144, 256, 1), (4096, 2048, 384, 1), (2048, 4096, 640, 1),          # enough full 256x256 tiles; 1, 2, 3, 5 k-tiles
    (256, 256, 256, 5), (512, 512, 512, 5), (1024, 1024, 1024, 5), (256, 768, 128, 5), (768, 256, 1152, 5),   # too few: 128-column tiles
    (64, 28672, 256, 5), (128, 40000, 128, 5), (90, 20000, 128, 5),      # one row tile: column pitch 112 / 128 / 80
    (48, 1024, 512, 5), (100, 3000, 256, 5), (129, 520, 384, 5), (256, 1000, 128, 5), (200, 136, 1280, 5), (33, 256, 256, 5),
    (64, 256, 128 * 7, 5), (40, 300, 128 * 12, 5), (96, 264, 128 * 9, 5), (80, 1024, 2048, 5), (128, 512, 128 * 11, 5),  # k-tiles issued in pairs
    (1000, 1000, 1024, 5), (300, 200, 256, 5), (257, 255, 128, 5), (32, 64, 8192 + 128, 5), (255, 1, 128, 5),
    (16, 512, 1024, 2), (1, 16, 128, 2), (5, 48, 256, 2), (16, 1000, 384, 2), (9, 33, 8192 + 128, 2), (16, 64, 16384, 2),
    (17, 256, 256, 2), (32, 512, 8192, 2), (24, 100, 1152, 2), (31, 33, 384, 2),        # two 16-row blocks on the skinny kernel
    (4000, 4100, 256, 3), (3000, 5000, 128, 3),                                          # ragged M, N on the 256x256 kernel
    (256, 256, 208, 3), (300, 200, 144, 3), (1000, 1000, 1040, 3), (64, 64, 16, 3), (16, 512, 1024 + 16, 3), (512, 256, 128 * 5 + 112, 3),  # K tails
    (100, 70, 50, 0), (256, 256, 200, 0), (3, 5, 7, 0), (64, 64, 0, 0),
])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_shapes_vs_oracle(m, n, k, path, out_dtype):
    assert _path(m, n, k) == path
    a, b, sa, sb = inputs.gemm_scaled(m, n, k, seed=m + 31 * n + 7 * k)
    out = hx.fp8_gemm(a.to(DEV), b.to(DEV), scale_a=sa.to(DEV), scale_b=sb.to(DEV), out_dtype=out_dtype)
    assert out.dtype == out_dtype and out.shape == (m, n)
    ref = orc.fp8_gemm(a, b, sa, sb, out_dtype)
    assert rel_err(out, ref) <= (1e-2 if out_dtype != torch.float32 else 1e-4)


@pytest.mark.parametrize("m,k,n,path,ws", [
    (256, 384, 512, 4, 0),            # tile kernel reads the row-major B in place (transposing LDS loads)
    (512, 1024, 768, 4, 0),
    (300, 256, 208, 4, 0),            # ragged M and N (N % 16 == 0): clamped chunks, guarded stores
    (1000, 512, 1008, 4, 0),
    (17, 128, 16, 4, 0),              # one valid 16-byte chunk per row
    (256, 400, 512, 4, 0),            # K % 128 != 0: the last k-tile is zero-padded in LDS
    (300, 144, 208, 4, 0),
    (100, 16, 48, 4, 0),
    (300, 256, 200, 0, 200 * 256),    # N % 16 != 0: transposed into the workspace, then the edge-tile kernel
    (16, 1024, 512, 0, 512 * 1024),   # skinny shape: transposed, then the skinny kernel
    (64, 100, 48, 0, 0),              # K % 128 != 0: general kernel
])
def test_row_major_b(m, k, n, path, ws):
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).to(E4M3); y = torch.randn(k, n, generator=g).to(E4M3)  # y row-major
    lib = _lib.load()
    xd, yd = x.to(DEV), y.to(DEV)
    assert lib.hx_fp8_gemm_path(m, n, k, k, n, 1, n, xd.data_ptr(), yd.data_ptr(), xd.data_ptr()) == path
    assert lib.hx_fp8_gemm_workspace_bytes(m, n, k, n, 1) == ws
    for od, tol in ((torch.float32, 1e-4), (torch.bfloat16, 1e-2)):
        out = hx.fp8_gemm(xd, yd, out_dtype=od)
        assert rel_err(out, orc.fp8_gemm(x, y, out_dtype=od)) <= tol
    # the same arithmetic as the column-major path: identical bits
    assert torch.equal(hx.fp8_gemm(xd, yd, out_dtype=torch.float32), hx.fp8_gemm(xd, yd.T.contiguous().T, out_dtype=torch.float32))
    # a strided (non-compact) row-major view works too
    ybig = torch.randn(k, n + 16, generator=g).to(E4M3)
    out2 = hx.fp8_gemm(xd, ybig.to(DEV)[:, :n], out_dtype=torch.float32)
    assert rel_err(out2, orc.fp8_gemm(x, ybig[:, :n].contiguous(), out_dtype=torch.float32)) <= 1e-4


def test_row_major_b_at_benchmark_size_matches_column_major():
    a, b, sa, sb = inputs.gemm_c2(DEV)
    b_row = b.contiguous()                       # [K, N] row-major copy of the column-major operand
    assert b_row.stride() == (8192, 1) and b.stride() == (1, 8192)
    out_col = hx.fp8_gemm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
    out_row = hx.fp8_gemm(a, b_row, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
    assert torch.equal(out_col, out_row)


def test_reference_call_form_and_defaults():
    # examples/fp8_gemm.py:95-109: randn -> e4m3, row-major y, fp16 result, unit scales
    g = torch.Generator().manual_seed(0)
    for m, k, n in [(256, 256, 256), (512, 512, 512)]:
        x = torch.randn(m, k, generator=g).to(E4M3); y = torch.randn(k, n, generator=g).to(E4M3)
        out = hx.fp8_gemm(x.to(DEV), y.to(DEV))
        assert out.dtype == torch.float16
        assert rel_err(out, orc.fp8_gemm(x, y)) <= 1e-2
        base = hx.reference_fp8_gemm_pytorch(x.to(DEV), y.to(DEV))
        torch.testing.assert_close(out.float(), base.float(), rtol=1e-2, atol=1e-1)  # helion/_testing.py:376-381
        assert torch.equal(hx.fp8_gemm_tritonbench(x.to(DEV), y.to(DEV)), out)


@pytest.mark.parametrize("m,n,k", [
    (300, 520, 2048),      # 128-row tiles, two splits
    (64, 2050, 2048),      # one 64-row tile, N % 4 != 0: scalar partial stores and reduce
    (33, 256, 128 * 17),   # 17 k-tiles in pieces of 9 and 8
    (200, 136, 4096),      # one 256-row tile
    (1024, 1280, 8192),    # three splits of 22, 22, 20 k-tiles
])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_split_k_few_tiles_long_k(m, n, k, out_dtype):
    """Few 128-column tiles and a long K: the op hands over the workspace that hx_fp8_gemm_workspace_bytes asks for
    and the kernel splits K (fp32 partial sums + reduce); without a workspace the same call runs unsplit."""
    lib = _lib.load()
    assert _path(m, n, k) == 5
    ws_bytes = lib.hx_fp8_gemm_workspace_bytes(m, n, k, 1, k)
    assert ws_bytes >= 2 * m * n * 4 and ws_bytes % (m * n * 4) == 0
    a, b, sa, sb = inputs.gemm_scaled(m, n, k, seed=m + n + k)
    ad, bd, sad, sbd = a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV)
    ref = orc.fp8_gemm(a, b, sa, sb, out_dtype)
    tol = 1e-2 if out_dtype != torch.float32 else 1e-4
    out = hx.fp8_gemm(ad, bd, scale_a=sad, scale_b=sbd, out_dtype=out_dtype)
    assert rel_err(out, ref) <= tol
    unsplit = torch.empty_like(out)
    rc = lib.hx_fp8_gemm(ad.data_ptr(), bd.data_ptr(), unsplit.data_ptr(), m, n, k, k, 1, k, n, sad.data_ptr(), sbd.data_ptr(),
                         _lib.HX_BF16 if out_dtype == torch.bfloat16 else _lib.HX_F32, None, 0,
                         torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.hx_last_error()
    assert rel_err(unsplit, ref) <= tol


def test_golden_fixture():
    z = np.load(G / "fp8_gemm_small.npz")
    for name in ("ragged", "skinny"):
        x = torch.from_numpy(z[f"{name}_x"].copy()).view(E4M3).to(DEV)
        yt = torch.from_numpy(z[f"{name}_yt"].copy()).view(E4M3).to(DEV)
        sa, sb = (torch.tensor(float(s), device=DEV) for s in z[f"{name}_scales"])
        out = hx.fp8_gemm(x, yt.T, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
        ref = torch.from_numpy(z[f"{name}_out_bf16"].copy()).view(torch.bfloat16)
        assert rel_err(out, ref) <= 1e-2
        ref16 = torch.from_numpy(z[f"{name}_out_f16_unit"].copy()).view(torch.float16)
        assert rel_err(hx.fp8_gemm(x, yt.T), ref16) <= 1e-2


def test_direct_c_abi_call_with_padded_leading_dimensions():
    lib = _lib.load()
    m, n, k, lda, ldb, ldc = 256, 512, 384, 512, 400, 520
    g = torch.Generator().manual_seed(3)
    abuf = torch.randn(m, lda, generator=g).to(E4M3); bbuf = torch.randn(n, ldb, generator=g).to(E4M3)
    ad, bd = abuf.to(DEV), bbuf.to(DEV)
    cd = torch.full((m, ldc), 7.0, dtype=torch.bfloat16, device=DEV)
    rc = lib.hx_fp8_gemm(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), m, n, k, lda, 1, ldb, ldc, None, None, _lib.HX_BF16,
                         None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.hx_last_error()
    torch.cuda.synchronize()
    ref = orc.fp8_gemm(abuf[:, :k], bbuf[:, :k].T, out_dtype=torch.bfloat16)
    assert rel_err(cd[:, :n], ref) <= 1e-2
    assert bool((cd[:, n:] == 7.0).all())  # padding columns untouched


def test_noncontiguous_x_and_nan_propagation():
    g = torch.Generator().manual_seed(4)
    big = torch.randn(64, 512, generator=g).to(E4M3)
    x = big[:, ::2]  # stride 2 along k -> the op makes it contiguous
    y = torch.randn(256, 128, generator=g).to(E4M3)
    out = hx.fp8_gemm(x.to(DEV), y.to(DEV), out_dtype=torch.float32)
    assert rel_err(out, orc.fp8_gemm(x.contiguous(), y, out_dtype=torch.float32)) <= 1e-4
    xn = torch.randn(256, 256, generator=g).to(E4M3); yn = torch.randn(256, 256, generator=g).to(E4M3)
    xb = xn.view(torch.uint8).clone(); xb[5, 17] = 0x7F
    xn = xb.view(E4M3)
    out = hx.fp8_gemm(xn.to(DEV), yn.T.contiguous().T.to(DEV), out_dtype=torch.float32).cpu()
    assert bool(torch.isnan(out[5]).all()) and not bool(torch.isnan(out[[0, 4, 6, 255]]).any())


def test_linearity_in_power_of_two_scales():
    a, b, sa, sb = inputs.gemm_scaled(256, 256, 512, 9, DEV)
    o1 = hx.fp8_gemm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.float32)
    o2 = hx.fp8_gemm(a, b, scale_a=sa * 2, scale_b=sb * 4, out_dtype=torch.float32)
    assert torch.equal(o2, o1 * 8)
    assert torch.equal(hx.fp8_gemm(a, b, out_dtype=torch.float32), hx.fp8_gemm(a, b, out_dtype=torch.float32))  # deterministic


def test_c1_1024_cube_matches_ref_eager_form():
    a, b = inputs.gemm_c1()
    out = hx.fp8_gemm(a.to(DEV), b.to(DEV), out_dtype=torch.bfloat16)
    ref = orc.fp8_gemm(a, b, out_dtype=torch.bfloat16)
    assert rel_err(out, ref) <= 1e-2


def test_c3_decode_shape_full_oracle():
    a, b, sa, sb = inputs.gemm_c3()
    assert _path(16, 28672, 8192) == 2
    out = hx.fp8_gemm(a.to(DEV), b.to(DEV), scale_a=sa.to(DEV), scale_b=sb.to(DEV), out_dtype=torch.bfloat16)
    ref = orc.fp8_gemm(a, b, sa, sb, torch.bfloat16)
    assert rel_err(out, ref) <= 1e-2


@pytest.mark.parametrize("m,n,k", [
    (16, 4096 + 16 * 37, 1024), (1, 8208, 2048), (16, 6000, 3072), (7, 4112, 5120), (16, 9000, 7168), (16, 12304, 8192),
    (24, 5008, 4096), (32, 4128, 8192), (16, 5000, 1152), (20, 4500, 8192 - 128),
    (16, 16 * 256 * 12, 1024), (3, 16 * 256 * 13 + 40, 2048), (16, 16 * 256 * 12 + 16, 1152),   # enough groups for tickets
])
def test_decode_kernel_more_column_groups_than_workgroups(m, n, k):
    """Every k-steps-per-wave variant of the decode kernel with column groups handed out by ticket (16-row variant) or by
    stride (32-row variant), against the oracle."""
    assert _path(m, n, k) == 2
    a, b, sa, sb = inputs.gemm_scaled(m, n, k, seed=n + k)
    out = hx.fp8_gemm(a.to(DEV), b.to(DEV), scale_a=sa.to(DEV), scale_b=sb.to(DEV), out_dtype=torch.float32)
    assert rel_err(out, orc.fp8_gemm(a, b, sa, sb, torch.float32)) <= 1e-4


def test_decode_kernel_ticket_word_needs_no_initialisation_and_is_left_clear():
    lib = _lib.load()
    m, n, k = 16, 16 * 256 * 12 + 16 * 100 + 5, 2048
    assert lib.hx_fp8_gemm_workspace_bytes(m, n, k, 1, k) >= 8
    a, b, sa, sb = inputs.gemm_scaled(m, n, k, seed=11)
    ad, bd = a.to(DEV), b.T.contiguous().to(DEV)   # [N][K]: the column-major B the kernel reads
    stream = torch.cuda.current_stream().cuda_stream

    def run(ws):
        c = torch.zeros((m, n), dtype=torch.float32, device=DEV)
        rc = lib.hx_fp8_gemm(ad.data_ptr(), bd.data_ptr(), c.data_ptr(), m, n, k, k, 1, k, n, None, None, _lib.HX_F32,
                             ws.data_ptr() if ws is not None else None, ws.numel() * 8 if ws is not None else 0, stream)
        assert rc == 0, lib.hx_last_error()
        torch.cuda.synchronize()
        return c

    static = run(None)                      # no workspace: strided shares, no tickets
    assert rel_err(static, orc.fp8_gemm(a, b, out_dtype=torch.float32)) <= 1e-4
    for fill in (-1, 0x7fffffffffffffff, 0x0123456789abcdef, 1, (5 << 24) | 77):   # stale contents of any kind
        ws = torch.full((2,), fill, dtype=torch.int64, device=DEV)
        assert torch.equal(run(ws), static)
        assert int(ws[0].item()) == 0       # the last draw clears the word ...
        assert torch.equal(run(ws), static)  # ... and a launch that finds it clear works as well
        assert int(ws[0].item()) == 0 and int(ws[1].item()) == fill


def test_c2_8192_cube_sampled_rows_and_checksum():
    a, b, sa, sb = inputs.gemm_c2()
    ad, bd = a.to(DEV), b.to(DEV)
    out = hx.fp8_gemm(ad, bd, scale_a=sa.to(DEV), scale_b=sb.to(DEV), out_dtype=torch.bfloat16)
    rows = torch.arange(0, 8192, 67)  # 123 rows spread over every row tile
    ref = orc.fp8_gemm(a[rows], b, sa, sb, torch.bfloat16)
    assert rel_err(out[rows.to(DEV)], ref) <= 1e-2
    # checksum of checksums: sum_n C[m,n] == alpha * A[m,:] . (sum_n B[:,n]); bf16 rounding noise averages out
    alpha = float(sa) * float(sb)
    bsum = orc.dq(b.T.contiguous()).double().sum(0)  # [K]
    expect = (orc.dq(a).double() @ bsum) * alpha
    got = out.double().sum(1).cpu()
    scale = (orc.dq(a).double().abs() @ orc.dq(b.T.contiguous()).double().abs().sum(0)) * alpha
    assert float(((got - expect).abs() / scale).max()) < 1e-4


def test_random_shapes_layouts_and_dtypes_vs_oracle():
    """A seeded sweep over shapes that land on every kernel (tile, edge tile, row-major B in place, skinny with one or
    two row blocks, transpose-through-workspace, general) and over both B layouts and all output types."""
    rng = np.random.default_rng(1234)
    lib = _lib.load()
    seen = set()
    for case in range(64):
        m = int(rng.choice([1, 7, 16, 17, 32, 33, 100, 256, 300, 513]))
        n = int(rng.choice([16, 48, 100, 256, 272, 400, 512, 1000]))
        k = int(rng.choice([128, 256, 384, 1024, 200, 16, 144, 1200]))
        row_major = bool(rng.integers(0, 2))
        od = [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(0, 3))]
        g = torch.Generator().manual_seed(case)
        x = (torch.randn(m, k, generator=g) * 0.7).to(E4M3)
        y = (torch.randn(k, n, generator=g) * 0.7).to(E4M3)            # row-major [K, N]
        yd = y.to(DEV) if row_major else y.to(DEV).T.contiguous().T      # or column-major with the same values
        sa = torch.rand((), generator=g) * 1.5 + 0.5; sb = torch.rand((), generator=g) * 1.5 + 0.5
        xd = x.to(DEV)
        seen.add(lib.hx_fp8_gemm_path(m, n, k, k, yd.stride(0), yd.stride(1), n, xd.data_ptr(), yd.data_ptr(), xd.data_ptr()))
        out = hx.fp8_gemm(xd, yd, scale_a=sa.to(DEV), scale_b=sb.to(DEV), out_dtype=od)
        ref = orc.fp8_gemm(x, y, sa, sb, od)
        assert rel_err(out, ref) <= (1e-2 if od != torch.float32 else 1e-4), (case, m, n, k, row_major, od)
    assert seen >= {0, 2, 3, 4, 5}   # the aligned 256x256 tile path (1) has its own cases above
