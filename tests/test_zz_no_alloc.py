"""hx_moe_grouped_gemm_static (the entry point that allocates nothing: its tile table and row flags live in a device
array built into the library) against hx_moe_grouped_gemm with a caller-provided workspace, both called through the
raw C ABI on the same inputs.  The two share their kernels, so the outputs must be identical bit for bit.  Two calls
in a row, the second on a smaller input, so that whatever the first call left in the shared array is seen to be
harmless; then the size limits."""
import pytest
import torch

from helion_amd import _lib, inputs
from helion_amd._lib import HX_BF16, HX_F16

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _tables(ex, E):
    idx = torch.argsort(ex, stable=True).to(torch.int32)
    counts = torch.bincount(ex, minlength=E).to(torch.int32)
    offsets = torch.zeros(E + 1, dtype=torch.int32, device=ex.device)
    offsets[1:] = torch.cumsum(counts, 0)
    return counts, offsets, idx


def _both(T, K, N, E, dtype, seed, poison, path):
    lib = _lib.load()
    A, W, ex = inputs.moe_inputs(T, K, N, E, 1, seed=seed, dtype=dtype)
    A, W, ex = A.to(DEV), W.to(DEV), ex.to(DEV)
    assert lib.hx_moe_path(T, K, N, E, 1, A.data_ptr(), W.data_ptr(), A.data_ptr()) == path  # the kernel this case is meant for
    if E > 2:
        ex[ex == 1] = 0  # an empty expert
    counts, offsets, idx = _tables(ex, E)
    counts[E - 1] = 0  # the last expert switched off: its rows are covered by nobody and must come out zero
    tag = HX_BF16 if dtype == torch.bfloat16 else HX_F16
    stream = torch.cuda.current_stream().cuda_stream
    ws_bytes = lib.hx_moe_workspace_bytes(T, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    ref = torch.full((T, N), poison, dtype=dtype, device=DEV)
    out = torch.full((T, N), poison, dtype=dtype, device=DEV)
    mt = int(counts.max().item())
    print(f"no-alloc case T={T} K={K} N={N} E={E} {dtype} seed={seed}", flush=True)
    rc = lib.hx_moe_grouped_gemm(A.data_ptr(), W.data_ptr(), ref.data_ptr(), counts.data_ptr(), offsets.data_ptr(), idx.data_ptr(),
                                 T, K, N, E, mt, tag, ws.data_ptr(), ws_bytes, stream)
    _lib.check(rc, "hx_moe_grouped_gemm")
    rc = lib.hx_moe_grouped_gemm_static(A.data_ptr(), W.data_ptr(), out.data_ptr(), counts.data_ptr(), offsets.data_ptr(),
                                        idx.data_ptr(), T, K, N, E, mt, tag, stream)
    _lib.check(rc, "hx_moe_grouped_gemm_static")
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), "static-scratch result differs from the workspace one"
    assert bool((out[ex == E - 1] == 0).all())
    assert bool(out.float().abs().max() > 0)
    return out


def test_two_calls_in_a_row_second_smaller():
    # first call: 128-row MFMA tiles, two-launch table build (T > 4096); second: fewer rows, fewer experts, the one-launch
    # table build -- it reads only what it wrote itself into the shared array
    _both(6000, 256, 512, 8, torch.bfloat16, seed=11, poison=3.0, path=2)
    _both(700, 128, 264, 5, torch.float16, seed=12, poison=-2.0, path=2)
    # a larger one again: the reference's own check shape, K = 500 (rows of A only 4-byte aligned): the 128-row MFMA
    # tiles with a partial last k-tile and A fetched in 4-byte pieces
    _both(1000, 500, 200, 30, torch.float16, seed=13, poison=1.0, path=5)
    # and an odd K, which only the fp32-FMA kernel takes
    _both(900, 251, 200, 6, torch.float16, seed=14, poison=-1.0, path=0)


def test_rejects_sizes_beyond_the_built_in_scratch():
    lib = _lib.load()
    d = torch.zeros(16, dtype=torch.int32, device=DEV)
    p = d.data_ptr()
    rc = lib.hx_moe_grouped_gemm_static(p, p, p, p, p, p, 131072 + 1, 64, 64, 4, 0, HX_BF16, None)
    assert rc == -2 and b"exceed" in lib.hx_last_error()
    rc = lib.hx_moe_grouped_gemm_static(p, p, p, p, p, p, 1024, 64, 64, 1025, 0, HX_BF16, None)
    assert rc == -2
    # empty problems return before anything is touched
    assert lib.hx_moe_grouped_gemm_static(None, None, None, None, None, None, 0, 64, 64, 4, 0, HX_BF16, None) == 0
