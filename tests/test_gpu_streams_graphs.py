"""The C ABI launches on the caller's stream and never allocates or synchronises, so the ops must work on a side
stream and inside a captured HIP graph.  Every replay is compared with the eager result, with eager work and
synchronisations between the replays."""
import pytest
import torch

import helion_amd as hx
from helion_amd import inputs

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _cases():
    a, b, sa, sb = inputs.gemm_scaled(512, 768, 256, seed=1)
    a, b, sa, sb = a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV)
    q, k, v = (t.to(DEV) for t in inputs.attention_inputs(1, 4, 256, 128, seed=2))
    A, W, ex = inputs.moe_inputs(300, 128, 256, 6, 2, seed=3)
    A, W, ex = A.to(DEV), W.to(DEV), ex.to(DEV)
    x = torch.randn(1000, 333, device=DEV, dtype=torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(4)
    mx = torch.randn(300, 1024, device=DEV, generator=g).to(torch.float16)
    my = torch.randn(1024, 264, device=DEV, generator=g).to(torch.float16)
    mb = torch.randn(264, device=DEV, generator=g).to(torch.float16)
    aq, ak, av = (torch.randn(2, 3, 200, 128, device=DEV, generator=g).to(torch.bfloat16) for _ in range(3))
    from helion_amd.matmul import bias_relu
    da, db, _, _ = inputs.gemm_scaled(16, 16 * 256 * 12, 1024, seed=6)      # enough column groups for the ticket hand-out
    da, db = da.to(DEV), db.to(DEV)
    A4, W4, ex4 = (t.to(DEV) for t in inputs.moe_inputs(200, 500, 72, 5, 1, seed=7, dtype=torch.float16))   # A by 4-byte DMA
    args4 = hx.moe_matmul_ogs_helion_kernel_args_gen(A4, W4, ex4)   # (has the reference's host sync: outside the capture)
    return {
        "fp8_gemm_decode_tickets": lambda: hx.fp8_gemm(da, db, out_dtype=torch.float32),
        "fp8_attention_ragged": lambda: hx.fp8_attention_kernel(q[:, :200].contiguous(), k[:, :200].contiguous(),
                                                                v[:, :, :200].contiguous(), 1, 4, out_dtype=torch.float32),
        "moe_partial_k_tile": lambda: hx.moe_matmul_ogs(*args4),
        "matmul_bias_relu": lambda: hx.matmul(mx, my, bias_relu(mb)),
        "matmul_split_k": lambda: hx.matmul_split_k(mx, my, split_k=4),
        "attention16": lambda: hx.attention(aq, ak, av),
        "attention16_ragged_keys": lambda: hx.attention(aq, ak[:, :, :150], av[:, :, :150]),
        "fp8_attention_plain": lambda: hx.fp8_attention_kernel(q[:, :100], k[:, :100], v[:, :, :100], 1, 4, out_dtype=torch.float32),
        "fp8_gemm": lambda: hx.fp8_gemm(a, b, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16),
        "fp8_gemm_row_major": lambda: hx.fp8_gemm(a, b.contiguous(), out_dtype=torch.float32),
        "fp8_gemm_skinny": lambda: hx.fp8_gemm(a[:16], b, out_dtype=torch.float32),
        "fp8_attention": lambda: hx.fp8_attention_kernel(q, k, v, 1, 4, out_dtype=torch.float32),
        "fp8_attention_online": lambda: hx.fp8_attention_kernel(q, k, v, 1, 4, out_dtype=torch.float32, exact_max=False),
        "moe_topk": lambda: hx.moe_matmul_topk(A[::2].contiguous(), W, ex, 2),
        "quantize": lambda: hx.fp8_quantize_per_tensor(x)[0].view(torch.uint8),
    }


def test_side_stream_matches_default_stream():
    cases = _cases()
    want = {n: f().clone() for n, f in cases.items()}
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = {n: f() for n, f in cases.items()}
    side.synchronize()
    for n in cases:
        assert torch.equal(got[n], want[n]), n


def test_graph_capture_and_replay():
    cases = _cases()
    want = {n: f().clone() for n, f in cases.items()}
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, as torch's graph recipe asks
        for f in cases.values():
            f()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = {n: f() for n, f in cases.items()}
    for replay in range(3):
        for o in outs.values():
            o.zero_()                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for n in cases:
            assert torch.equal(outs[n], want[n]), (n, replay)


def test_entry_points_trace_under_torch_compile():
    """In eager mode the entry points call the implementation directly; while tracing they go through the registered
    ops (shape inference on fake tensors).  Dynamo with the pass-through backend: no code generation involved."""
    cases = _cases()
    for name in ("fp8_gemm", "matmul_bias_relu", "attention16", "fp8_attention"):
        fn = cases[name]
        want = fn()
        got = torch.compile(fn, backend="eager", fullgraph=True)()
        assert torch.equal(got, want), name
