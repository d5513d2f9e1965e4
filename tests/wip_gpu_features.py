"""GPU parity of the opt-in kernel paths (helion_amd.set_features).  NOT collected by pytest on purpose (the file name
does not start with test_): these paths have passed the CPU-side checks in the host execution model but have never run on
an MI355X.  Run it by naming the file:  python -m pytest tests/wip_gpu_features.py -x -q --timeout 120
and rename it to test_gpu_features.py once it passes there."""
import pytest
import torch

import helion_amd as hx
from helion_amd import _lib
from oracle import oracle as orc
from tests._util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"
E4 = torch.float8_e4m3fn


@pytest.fixture
def rowmajor_decode():
    old = hx.set_features(hx.HX_FEATURE_SKINNY_ROWMAJOR)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("m,n,k,od", [(16, 256, 1024, torch.bfloat16), (1, 16, 1024, torch.float16), (7, 144, 2048, torch.bfloat16),
                                      (16, 2048, 4096, torch.bfloat16), (32, 384, 8192, torch.bfloat16), (20, 640, 1024, torch.float32),
                                      (16, 40000, 1024, torch.bfloat16), (16, 28672, 8192, torch.bfloat16)])
def test_rowmajor_decode_kernel(rowmajor_decode, m, n, k, od):
    g = torch.Generator().manual_seed(m + n + k)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4)
    y = (torch.randn(k, n, generator=g) * 0.5).to(E4)
    sa, sb = torch.tensor(1.5), torch.tensor(0.5)
    lib = _lib.load()
    ad, yd = a.to(DEV), y.to(DEV)
    assert lib.hx_fp8_gemm_path(m, n, k, k, n, 1, n, ad.data_ptr(), yd.data_ptr(), ad.data_ptr()) == 6
    print(f"rowmajor decode case M={m} N={n} K={k} {od}", flush=True)
    out = hx.fp8_gemm(ad, yd, scale_a=sa.to(DEV), scale_b=sb.to(DEV), out_dtype=od)
    assert rel_err(out, orc.fp8_gemm(a, y, 1.5, 0.5, od)) <= 1e-2


@pytest.fixture
def any_k():
    old = hx.set_features(hx.HX_FEATURE_FP8_GEMM_ANY_K)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("m,n,k,rowmajor", [(300, 260, 1000, False), (33, 100, 1001, False), (16, 512, 2047, False), (64, 1792, 1023, False),
                                            (200, 272, 100, True), (5, 7, 24, False), (256, 256, 3, True), (2048, 2048, 4100, False)])
def test_any_k_through_the_mfma_kernels(any_k, m, n, k, rowmajor):
    g = torch.Generator().manual_seed(77 + k)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4)
    bt = (torch.randn(n, k, generator=g) * 0.5).to(E4)
    y = bt.t().contiguous() if rowmajor else bt.t()
    print(f"any-K case M={m} N={n} K={k} rowmajor={rowmajor}", flush=True)
    out = hx.fp8_gemm(a.to(DEV), y.to(DEV), out_dtype=torch.bfloat16)
    assert rel_err(out, orc.fp8_gemm(a, y, 1.0, 1.0, torch.bfloat16)) <= 1e-2


@pytest.fixture
def d256():
    old = hx.set_features(hx.HX_FEATURE_ATTENTION_D256)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("s,d,exact,strided_v", [(64, 256, True, False), (208, 256, True, True), (640, 256, False, False), (1104, 256, True, False),
                                                 (331, 256, False, True), (500, 192, True, False), (4096, 256, True, False)])
def test_attention_head_dim_256(d256, s, d, exact, strided_v):
    g = torch.Generator().manual_seed(s + d)
    q, k = (torch.randn(2, s, d, generator=g).to(E4) for _ in range(2))
    v = torch.randn(2, d, s, generator=g).to(E4)
    vd = v.to(DEV)
    if strided_v:
        vd = vd.transpose(1, 2).contiguous().transpose(1, 2)
    print(f"attention D256 case S={s} D={d} exact={exact} strided_v={strided_v}", flush=True)
    out = hx.fp8_attention_kernel(q.to(DEV), k.to(DEV), vd, 1, 2, out_dtype=torch.float32, exact_max=exact)
    ref = orc.fp8_attention(q, k, v, 1, 2, torch.float32) if exact else orc.fp8_attention_tiled(q, k, v, 1, 2, 64, torch.float32)
    assert rel_err(out, ref) <= 3e-2


@pytest.fixture
def persistent():
    old = hx.set_features(hx.HX_FEATURE_FP8_GEMM_PERSISTENT)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("m,n,k,od", [(8192, 8192, 512, torch.bfloat16), (8192, 4096, 1024, torch.float16), (5888, 8192, 768, torch.bfloat16),
                                      (8192, 8192, 8192, torch.bfloat16)])
def test_persistent_256_tile_kernel(persistent, m, n, k, od):
    """Bit-equal to the default 256x256 kernel (same MFMA order per accumulator), and within tolerance of the oracle on
    the rows the CPU finishes in seconds."""
    g = torch.Generator().manual_seed(m + n + k)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4).to(DEV)
    bt = (torch.randn(n, k, generator=g) * 0.5).to(E4).to(DEV)
    sa, sb = torch.tensor(1.25, device=DEV), torch.tensor(0.5, device=DEV)
    lib = _lib.load()
    assert lib.hx_fp8_gemm_path(m, n, k, k, 1, k, n, a.data_ptr(), bt.data_ptr(), a.data_ptr()) == 7
    print(f"persistent case M={m} N={n} K={k} {od}", flush=True)
    out = hx.fp8_gemm(a, bt.t(), scale_a=sa, scale_b=sb, out_dtype=od)
    hx.set_features(0)
    base = hx.fp8_gemm(a, bt.t(), scale_a=sa, scale_b=sb, out_dtype=od)
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    rows = torch.arange(0, m, 131)
    ref = orc.fp8_gemm(a[rows.to(DEV)].cpu(), bt.t().cpu(), 1.25, 0.5, od)
    assert rel_err(out[rows.to(DEV)].cpu(), ref) <= 1e-2


@pytest.fixture
def decode_ring():
    old = hx.set_features(hx.HX_FEATURE_FP8_GEMM_DECODE_RING)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("m,n,k,od", [(33, 100, 128, torch.bfloat16), (64, 256, 2560, torch.bfloat16), (128, 256, 2560, torch.float16),
                                      (100, 640, 512, torch.float32), (40, 512, 1024, torch.bfloat16), (96, 128, 8192, torch.bfloat16),
                                      (64, 28672, 8192, torch.bfloat16), (128, 28672, 8192, torch.bfloat16), (130, 256, 1024, torch.bfloat16),
                                      (200, 640, 512, torch.float16), (160, 28672, 8192, torch.bfloat16), (256, 28672, 8192, torch.bfloat16)])
def test_decode_ring_kernel(decode_ring, m, n, k, od):
    """Bit-equal to the kernel it replaces (hx_fp8_gemm_tileN128: same MFMA order), and within tolerance of the oracle."""
    g = torch.Generator().manual_seed(m + n + k)
    a = (torch.randn(m, k, generator=g) * 0.5).to(E4)
    bt = (torch.randn(n, k, generator=g) * 0.5).to(E4)
    ad, btd = a.to(DEV), bt.to(DEV)
    sa, sb = torch.tensor(1.25, device=DEV), torch.tensor(0.5, device=DEV)
    assert _lib.load().hx_fp8_gemm_path(m, n, k, k, 1, k, n, ad.data_ptr(), btd.data_ptr(), ad.data_ptr()) == 8
    print(f"decode ring case M={m} N={n} K={k} {od}", flush=True)
    out = hx.fp8_gemm(ad, btd.t(), scale_a=sa, scale_b=sb, out_dtype=od)
    hx.set_features(0)
    base = hx.fp8_gemm(ad, btd.t(), scale_a=sa, scale_b=sb, out_dtype=od)
    assert torch.equal(out.view(torch.uint8), base.view(torch.uint8))
    cols = torch.arange(0, n, max(1, n // 512))
    ref = orc.fp8_gemm(a, bt[cols].t(), 1.25, 0.5, od)
    assert rel_err(out[:, cols.to(DEV)].cpu(), ref) <= 1e-2


@pytest.fixture
def routing_wide():
    old = hx.set_features(hx.HX_FEATURE_ROUTING_WIDE)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("T,E,dtype", [(3000, 513, torch.int64), (20000, 2048, torch.int64), (70000, 2048, torch.int32), (1 << 20, 1024, torch.int64)])
def test_routing_tables_for_513_to_2048_experts(routing_wide, T, E, dtype):
    g = torch.Generator().manual_seed(T + E)
    ids = torch.randint(0, E, (T,), generator=g).to(dtype)
    print(f"wide routing case T={T} E={E} {dtype}", flush=True)
    counts, offsets, idx, mx = hx.moe_routing(ids.to(DEV), E)
    rc = torch.bincount(ids.long(), minlength=E).int()
    assert torch.equal(counts.cpu(), rc) and torch.equal(idx.cpu(), torch.argsort(ids.long(), stable=True).int())
    assert torch.equal(offsets.cpu()[1:], torch.cumsum(rc, 0).int()) and int(mx) == int(rc.max())


@pytest.fixture
def moe_persistent():
    old = hx.set_features(hx.HX_FEATURE_MOE_PERSISTENT)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("T,K,N,E,dtype", [(65536, 256, 2048, 4, torch.bfloat16), (65536, 384, 1024, 8, torch.float16),
                                           (40000, 1024, 4096, 3, torch.bfloat16), (65536, 4096, 14336, 8, torch.bfloat16)])
def test_persistent_grouped_gemm(moe_persistent, T, K, N, E, dtype):
    """Bit-equal to the default 256-row-tile kernel (same MFMA order per accumulator); a sample of rows against the oracle."""
    from helion_amd import inputs
    A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=T + K, dtype=dtype, device=DEV)
    lib = _lib.load()
    assert lib.hx_moe_path(T, K, N, E, 1, A.data_ptr(), W.data_ptr(), A.data_ptr()) == 6
    print(f"persistent grouped case T={T} K={K} N={N} E={E} {dtype}", flush=True)
    args = hx.moe_matmul_ogs_helion_kernel_args_gen(A, W, ex)
    out = hx.moe_matmul_ogs(*args)
    hx.set_features(0)
    base = hx.moe_matmul_ogs(*args)
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    rows = torch.arange(0, T, 997, device=DEV)
    ref = orc.moe_matmul_ogs_reference(A[rows].cpu(), W.cpu(), ex[rows].cpu())
    assert rel_err(out[rows].cpu(), ref) <= 1e-2


@pytest.fixture
def matmul_persistent():
    old = hx.set_features(hx.HX_FEATURE_MATMUL_PERSISTENT)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("m,n,k,dtype", [(8192, 8192, 256, torch.bfloat16), (8192, 16384, 384, torch.float16), (8192, 8192, 8192, torch.bfloat16)])
def test_persistent_dense_matmul(matmul_persistent, m, n, k, dtype):
    """Bit-equal to the default 256x256 kernel; a sample of rows against the oracle."""
    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn(m, k, generator=g) * 0.5).to(dtype).to(DEV)
    y = (torch.randn(k, n, generator=g) * 0.5).to(dtype).to(DEV)
    assert _lib.load().hx_matmul_path(m, n, k, k, n, 1, n, _lib.HX_BF16, x.data_ptr(), y.data_ptr(), x.data_ptr(), None) == 2
    print(f"persistent dense case M={m} N={n} K={k} {dtype}", flush=True)
    out = hx.matmul(x, y)
    hx.set_features(0)
    base = hx.matmul(x, y)
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    rows = torch.arange(0, m, 509, device=DEV)
    assert rel_err(out[rows].cpu(), orc.matmul(x[rows].cpu(), y.cpu())) <= 1e-2


@pytest.fixture
def moe_any_shape():
    old = hx.set_features(hx.HX_FEATURE_MOE_ANY_SHAPE)
    yield
    hx.set_features(old)


@pytest.mark.parametrize("T,K,N,E,dtype", [(37, 101, 24, 3, torch.bfloat16), (37, 100, 19, 3, torch.bfloat16), (300, 251, 203, 5, torch.float16),
                                           (600, 65, 260, 4, torch.bfloat16), (20, 1, 9, 2, torch.bfloat16), (5000, 1001, 1003, 8, torch.bfloat16)])
def test_moe_any_shape_through_the_mfma_kernels(moe_any_shape, T, K, N, E, dtype):
    from helion_amd import inputs
    A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=T + K + N, dtype=dtype)
    print(f"moe any-shape case T={T} K={K} N={N} E={E} {dtype}", flush=True)
    out = hx.moe_matmul_ogs(*hx.moe_matmul_ogs_helion_kernel_args_gen(A.to(DEV), W.to(DEV), ex.to(DEV)))
    assert rel_err(out.cpu(), orc.moe_matmul_ogs_reference(A, W, ex)) <= 1e-2
