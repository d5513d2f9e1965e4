"""torch.library registrations: each op validates, allocates the output (and workspace) with torch
and calls the C ABI on the current HIP stream.  Tensors are plumbing; the arithmetic is in
libhx_kernels.so."""
from __future__ import annotations

import torch

from . import _lib

_DT = {torch.float16: _lib.HX_F16, torch.bfloat16: _lib.HX_BF16, torch.float32: _lib.HX_F32,
       torch.float8_e4m3fn: _lib.HX_E4M3}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device: torch.device) -> int:
    """Handle of the current HIP stream of `device` (the raw getter skips building a Stream object: 2 us per call)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def eager(op_impl, op, *args):
    """Call the op's implementation directly for plain CUDA tensors in eager mode (the dispatcher round trip of a
    custom op costs more than a small kernel), and through the registered op when tracing / compiling or for anything
    else (fake or meta tensors get shape inference there, CPU tensors their error)."""
    if not torch.compiler.is_compiling() and all(type(a) is torch.Tensor and a.is_cuda for a in args if isinstance(a, torch.Tensor)):
        return op_impl(*args)
    return op(*args)


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("helion_amd ops run on the GPU only (HIP kernels); got a tensor on " + str(t.device))


# ------------------------------------------------------------------------------ fp8 gemm
def _fp8_gemm_impl(x: torch.Tensor, y: torch.Tensor, scale_a: torch.Tensor | None, scale_b: torch.Tensor | None,
                out_dtype: torch.dtype) -> torch.Tensor:
    _require_cuda(x, y, scale_a, scale_b)
    if x.dtype != torch.float8_e4m3fn or y.dtype != torch.float8_e4m3fn:
        raise TypeError(f"fp8_gemm expects float8_e4m3fn operands, got {x.dtype} and {y.dtype}")
    if x.dim() != 2 or y.dim() != 2:
        raise ValueError("fp8_gemm expects 2-D operands")
    m, k = x.shape
    k2, n = y.shape
    assert k == k2, f"size mismatch {k} != {k2}"
    if out_dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"unsupported out_dtype {out_dtype}")
    for s in (scale_a, scale_b):
        if s is not None and (s.dtype != torch.float32 or s.numel() != 1):
            raise TypeError("scales must be one-element float32 tensors")
    if x.stride(1) != 1 and k > 1:
        x = x.contiguous()
    lda = x.stride(0) if m > 1 else max(k, 1)
    if lda < k:
        x = x.contiguous()
        lda = k
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0 or n == 0:
        return out
    # B strides: (k stride, n stride); size-1 dims get the canonical stride
    ldb_k = y.stride(0) if k > 1 else 1
    ldb_n = y.stride(1) if n > 1 else max(k, 1)
    lib = _lib.load()
    ws_bytes = lib.hx_fp8_gemm_workspace_bytes(m, n, k, ldb_k, ldb_n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    rc = lib.hx_fp8_gemm(x.data_ptr(), y.data_ptr(), out.data_ptr(), m, n, k, lda, ldb_k, ldb_n, n,
                         scale_a.data_ptr() if scale_a is not None else None,
                         scale_b.data_ptr() if scale_b is not None else None,
                         _DT[out_dtype], ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x.device))
    _lib.check(rc, "hx_fp8_gemm")
    return out


fp8_gemm_op = torch.library.custom_op("helion_amd::fp8_gemm", mutates_args=())(_fp8_gemm_impl)


@fp8_gemm_op.register_fake
def _(x, y, scale_a, scale_b, out_dtype):
    return x.new_empty((x.shape[0], y.shape[1]), dtype=out_dtype)


# ------------------------------------------------------------------------------ fp8 attention
def _fp8_attention_impl(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, batch: int, heads: int,
                     out_dtype: torch.dtype, exact_max: int) -> torch.Tensor:
    _require_cuda(q, k, v)
    for t in (q, k, v):
        if t.dtype != torch.float8_e4m3fn:
            raise TypeError(f"fp8_attention expects float8_e4m3fn tensors, got {t.dtype}")
        if t.dim() != 3:
            raise ValueError("fp8_attention expects [batch*heads, seq, dim] / [batch*heads, dim, seq] tensors")
    bh, s, d = q.shape
    if bh != batch * heads:
        raise ValueError(f"q.size(0)={bh} != batch*heads={batch * heads}")
    if tuple(k.shape) != (bh, s, d) or tuple(v.shape) != (bh, d, s):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)} (v must be [BH, D, S])")
    if out_dtype not in (torch.float8_e4m3fn, torch.float32):
        raise TypeError(f"unsupported out_dtype {out_dtype}")
    d_true = d
    d256 = bool(_lib.load().hx_get_features() & _lib.HX_FEATURE_ATTENTION_D256)  # opt-in: head dim 256 on the MFMA kernel
    if d not in (64, 128) and 0 < d < 128 or (d256 and 128 < d < 256):
        # zero-pad the head dimension to what the MFMA kernel takes: q.k and the other output columns are unchanged,
        # the softmax scale still comes from the true head dimension
        dp = 64 if d < 64 else 128 if d < 128 else 256
        q = torch.nn.functional.pad(q.view(torch.uint8), (0, dp - d)).view(torch.float8_e4m3fn)
        k = torch.nn.functional.pad(k.view(torch.uint8), (0, dp - d)).view(torch.float8_e4m3fn)
        v = torch.nn.functional.pad(v.contiguous().view(torch.uint8), (0, 0, 0, dp - d)).view(torch.float8_e4m3fn)
        d = dp
    q, k = q.contiguous(), k.contiguous()
    # v is logically [BH, D, S].  The reference's preprocessing hands it over as a permuted view of [BH, S, D]
    # memory (strides (S*D, 1, D)); the kernel reads that layout directly, so only other stridings are copied.
    if bh > 1 and v.stride(0) != s * d or v.stride()[1:] not in ((s, 1), (1, d)):
        v = v.contiguous()
    if v.stride()[1:] == (s, 1) and s % 16 != 0 and d in (64, 128, 256) and s > 1:
        # [D][S] rows that are not a multiple of 16 bytes cannot be fetched in 16-byte pieces: hand the MFMA kernel the
        # [S][D] layout instead (one copy) rather than fall to the plain kernel
        v = v.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.empty((batch, heads, s, d), dtype=out_dtype, device=q.device)
    if bh == 0 or s == 0:
        return out
    lib = _lib.load()
    rc = lib.hx_fp8_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), bh, s, d, d_true, v.stride(1),
                              v.stride(2), _DT[out_dtype], int(exact_max), _stream_ptr(q.device))
    _lib.check(rc, "hx_fp8_attention")
    return out if d == d_true else out[..., :d_true].contiguous()


fp8_attention_op = torch.library.custom_op("helion_amd::fp8_attention", mutates_args=())(_fp8_attention_impl)


@fp8_attention_op.register_fake
def _(q, k, v, batch, heads, out_dtype, exact_max):
    return q.new_empty((batch, heads, q.shape[1], q.shape[2]), dtype=out_dtype)


# ------------------------------------------------------------------------------ moe grouped gemm
def _moe_matmul_ogs_impl(A: torch.Tensor, W: torch.Tensor, expert_token_counts: torch.Tensor,
                      expert_token_offsets: torch.Tensor, sorted_to_orig_token_idx: torch.Tensor,
                      max_T_per_expert: int) -> torch.Tensor:
    _require_cuda(A, W, expert_token_counts, expert_token_offsets, sorted_to_orig_token_idx)
    if A.dim() != 2 or W.dim() != 3:
        raise ValueError("moe_matmul_ogs expects A [T,K] and W [E,K,N]")
    T, K = A.shape
    E, K2, N = W.shape
    if K != K2:
        raise ValueError(f"size mismatch K={K} vs W.size(1)={K2}")
    dtype = torch.promote_types(A.dtype, W.dtype)
    if dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"moe_matmul_ogs supports float16/bfloat16, got {A.dtype} x {W.dtype}")
    A = A.to(dtype).contiguous()
    W = W.to(dtype).contiguous()
    counts = expert_token_counts.to(torch.int32).contiguous()
    offsets = expert_token_offsets.to(torch.int32).contiguous()
    idx = sorted_to_orig_token_idx.to(torch.int32).contiguous()
    if counts.numel() != E or offsets.numel() != E + 1 or idx.numel() != T:
        raise ValueError("routing tables must have shapes [E], [E+1], [T]")
    C = torch.empty((T, N), dtype=dtype, device=A.device)
    if T == 0 or N == 0:
        return C
    lib = _lib.load()
    ws_bytes = lib.hx_moe_workspace_bytes_shape(T, K, N, E)  # (= hx_moe_workspace_bytes(T, E) unless an opt-in path wants more)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=A.device)
    rc = lib.hx_moe_grouped_gemm(A.data_ptr(), W.data_ptr(), C.data_ptr(), counts.data_ptr(), offsets.data_ptr(),
                                 idx.data_ptr(), T, K, N, E, max_T_per_expert, _DT[dtype], ws.data_ptr(), ws_bytes,
                                 _stream_ptr(A.device))
    _lib.check(rc, "hx_moe_grouped_gemm")
    return C


moe_matmul_ogs_op = torch.library.custom_op("helion_amd::moe_matmul_ogs", mutates_args=())(_moe_matmul_ogs_impl)


@moe_matmul_ogs_op.register_fake
def _(A, W, expert_token_counts, expert_token_offsets, sorted_to_orig_token_idx, max_T_per_expert):
    return A.new_empty((A.shape[0], W.shape[2]), dtype=torch.promote_types(A.dtype, W.dtype))


# ------------------------------------------------------------------------------ moe routing tables
def _moe_routing_impl(expert_ids: torch.Tensor, num_experts: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(counts [E], offsets [E+1], idx [T], max_count [1]), all int32 on the device, no host synchronisation."""
    _require_cuda(expert_ids)
    if expert_ids.dim() != 1 or expert_ids.dtype not in (torch.int32, torch.int64):
        raise ValueError("moe_routing expects a 1-D int32 or int64 tensor of expert ids")
    ids = expert_ids.contiguous()
    T, E = ids.numel(), int(num_experts)
    dev = ids.device
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    idx = torch.empty(T, dtype=torch.int32, device=dev)
    max_count = torch.empty(1, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.hx_moe_routing_workspace_bytes(T, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    rc = lib.hx_moe_routing(ids.data_ptr(), int(ids.dtype == torch.int64), T, E, counts.data_ptr(), offsets.data_ptr(),
                            idx.data_ptr(), max_count.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes,
                            _stream_ptr(dev))
    _lib.check(rc, "hx_moe_routing")
    return counts, offsets, idx, max_count


moe_routing_op = torch.library.custom_op("helion_amd::moe_routing", mutates_args=())(_moe_routing_impl)


@moe_routing_op.register_fake
def _(expert_ids, num_experts):
    i32 = dict(dtype=torch.int32)
    return (expert_ids.new_empty(num_experts, **i32), expert_ids.new_empty(num_experts + 1, **i32),
            expert_ids.new_empty(expert_ids.shape[0], **i32), expert_ids.new_empty(1, **i32))


# ------------------------------------------------------------------------------ moe top-k matmul (routing fused in)
def _moe_matmul_topk_impl(A: torch.Tensor, W: torch.Tensor, expert_ids: torch.Tensor, top_k: int) -> torch.Tensor:
    _require_cuda(A, W, expert_ids)
    if A.dim() != 2 or W.dim() != 3:
        raise ValueError("moe_matmul_topk expects A [T_tok,K] and W [E,K,N]")
    T_tok, K = A.shape
    E, K2, N = W.shape
    if K != K2:
        raise ValueError(f"size mismatch K={K} vs W.size(1)={K2}")
    if top_k < 1 or expert_ids.numel() != T_tok * top_k:
        raise ValueError("expert_ids must hold T_tok * top_k ids (token-major)")
    if expert_ids.dtype not in (torch.int32, torch.int64):
        raise ValueError("expert_ids must be int32 or int64")
    dtype = torch.promote_types(A.dtype, W.dtype)
    if dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"moe_matmul_topk supports float16/bfloat16, got {A.dtype} x {W.dtype}")
    A = A.to(dtype).contiguous()
    W = W.to(dtype).contiguous()
    ids = expert_ids.reshape(-1).contiguous()
    C = torch.empty((T_tok * top_k, N), dtype=dtype, device=A.device)
    if C.numel() == 0:
        return C
    lib = _lib.load()
    ws_bytes = lib.hx_moe_topk_workspace_bytes(T_tok, top_k, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=A.device)
    rc = lib.hx_moe_topk_matmul(A.data_ptr(), W.data_ptr(), C.data_ptr(), ids.data_ptr(), int(ids.dtype == torch.int64),
                                T_tok, top_k, K, N, E, _DT[dtype], ws.data_ptr(), ws_bytes, _stream_ptr(A.device))
    _lib.check(rc, "hx_moe_topk_matmul")
    return C


moe_matmul_topk_op = torch.library.custom_op("helion_amd::moe_matmul_topk", mutates_args=())(_moe_matmul_topk_impl)


@moe_matmul_topk_op.register_fake
def _(A, W, expert_ids, top_k):
    return A.new_empty((A.shape[0] * top_k, W.shape[2]), dtype=torch.promote_types(A.dtype, W.dtype))


# ------------------------------------------------------------------------------ casts / quantisation in front of the fp8 kernels
def _cast_e4m3_x3_impl(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Three equally sized contiguous fp16/bf16/fp32 tensors -> e4m3 (same shapes), one launch."""
    _require_cuda(q, k, v)
    if not (q.dtype == k.dtype == v.dtype) or q.dtype not in _DT or q.dtype == torch.float8_e4m3fn:
        raise TypeError(f"cast_e4m3_x3 expects three float16/bfloat16/float32 tensors of one dtype, got {q.dtype}, {k.dtype}, {v.dtype}")
    if not (q.numel() == k.numel() == v.numel()):
        raise ValueError("cast_e4m3_x3 expects equally sized tensors")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    outs = [torch.empty(t.shape, dtype=torch.float8_e4m3fn, device=t.device) for t in (q, k, v)]
    lib = _lib.load()
    rc = lib.hx_fp8_attention_preprocess(q.data_ptr(), k.data_ptr(), v.data_ptr(), outs[0].data_ptr(), outs[1].data_ptr(),
                                         outs[2].data_ptr(), q.numel(), _DT[q.dtype], _stream_ptr(q.device))
    _lib.check(rc, "hx_fp8_attention_preprocess")
    return outs[0], outs[1], outs[2]


cast_e4m3_x3_op = torch.library.custom_op("helion_amd::cast_e4m3_x3", mutates_args=())(_cast_e4m3_x3_impl)


@cast_e4m3_x3_op.register_fake
def _(q, k, v):
    f8 = torch.float8_e4m3fn
    return q.new_empty(q.shape, dtype=f8), k.new_empty(k.shape, dtype=f8), v.new_empty(v.shape, dtype=f8)


def _fp8_quantize_impl(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """(e4m3 tensor of x's shape, 0-d fp32 scale) with x ~ q * scale; scale = max|x| / 448."""
    _require_cuda(x)
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"fp8_quantize expects float16/bfloat16/float32, got {x.dtype}")
    x = x.contiguous()
    q = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    ws_bytes = lib.hx_fp8_quantize_workspace_bytes(x.numel())
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    rc = lib.hx_fp8_quantize(x.data_ptr(), q.data_ptr(), x.numel(), _DT[x.dtype], scale.data_ptr(), ws.data_ptr(), ws_bytes,
                             _stream_ptr(x.device))
    _lib.check(rc, "hx_fp8_quantize")
    return q, scale


fp8_quantize_op = torch.library.custom_op("helion_amd::fp8_quantize", mutates_args=())(_fp8_quantize_impl)


@fp8_quantize_op.register_fake
def _(x):
    return x.new_empty(x.shape, dtype=torch.float8_e4m3fn), x.new_empty((), dtype=torch.float32)


# ------------------------------------------------------------------------------ dense matmul (+ bias, relu, split-K)
def _matmul_impl(x: torch.Tensor, y: torch.Tensor, bias: torch.Tensor | None, relu: bool, out_dtype: torch.dtype,
              split_k: int) -> torch.Tensor:
    _require_cuda(x, y, bias)
    if x.dim() != 2 or y.dim() != 2:
        raise ValueError("matmul expects 2-D operands")
    m, k = x.shape
    k2, n = y.shape
    assert k == k2, f"size mismatch {k} != {k2}"
    dt = torch.promote_types(x.dtype, y.dtype)
    if dt not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"matmul supports float16, bfloat16 and float32 operands, got {x.dtype} and {y.dtype}")
    if out_dtype not in (dt, torch.float32):
        raise TypeError(f"out_dtype must be {dt} or float32, got {out_dtype}")
    x = x.to(dt)
    y = y.to(dt)
    if k > 1 and x.stride(1) != 1 or (m > 1 and x.stride(0) < k):
        x = x.contiguous()
    lda = x.stride(0) if m > 1 else max(k, 1)
    if bias is not None:
        if bias.numel() != n:
            raise ValueError(f"bias must have {n} elements, got shape {tuple(bias.shape)}")
        bias = bias.reshape(n)
        if bias.dtype not in (dt, torch.float32):
            bias = bias.to(torch.float32)
        bias = bias.contiguous()
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0 or n == 0:
        return out
    ldb_k = y.stride(0) if k > 1 else max(n, 1)
    ldb_n = y.stride(1) if n > 1 else 1
    lib = _lib.load()
    has_ep = int(bias is not None or relu)
    ws_bytes = lib.hx_matmul_workspace_bytes(m, n, k, lda, ldb_k, ldb_n, n, _DT[dt], _DT[out_dtype], has_ep, split_k)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    rc = lib.hx_matmul(x.data_ptr(), y.data_ptr(), out.data_ptr(), m, n, k, lda, ldb_k, ldb_n, n,
                       bias.data_ptr() if bias is not None else None, _DT[bias.dtype] if bias is not None else 0,
                       int(relu), _DT[dt], _DT[out_dtype], split_k, ws.data_ptr() if ws is not None else None, ws_bytes,
                       _stream_ptr(x.device))
    _lib.check(rc, "hx_matmul")
    return out


matmul_op = torch.library.custom_op("helion_amd::matmul", mutates_args=())(_matmul_impl)


@matmul_op.register_fake
def _(x, y, bias, relu, out_dtype, split_k):
    return x.new_empty((x.shape[0], y.shape[1]), dtype=out_dtype)


# ------------------------------------------------------------------------------ 16-bit attention
def _attention_impl(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    _require_cuda(q, k, v)
    if q.dtype not in (torch.float16, torch.bfloat16, torch.float32) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError(f"attention expects q, k, v of one dtype out of float16, bfloat16, float32; got {q.dtype}, {k.dtype}, {v.dtype}")
    if q.dim() < 2 or k.dim() != q.dim() or v.dim() != q.dim():
        raise ValueError("attention expects q, k, v of shape [..., seq, head_dim] with the same number of dimensions")
    m_dim, d = q.shape[-2], q.shape[-1]
    n_dim = k.shape[-2]
    assert n_dim == v.shape[-2]
    assert d == k.shape[-1] == v.shape[-1]
    if n_dim == 0 and q.numel():
        raise ValueError("attention: no keys (softmax over an empty set)")
    if q.numel() == 0:
        return torch.empty_like(q, memory_format=torch.contiguous_format)
    q3, k3, v3 = q.reshape(-1, m_dim, d), k.reshape(-1, n_dim, d), v.reshape(-1, n_dim, d)
    bh = q3.shape[0]
    if k3.shape[0] != bh or v3.shape[0] != bh:
        raise ValueError("attention: q, k, v disagree on the batch dimensions")
    dp = d
    if q.dtype != torch.float32 and d not in (64, 128) and d < 128:
        # zero-pad the head dimension to what the MFMA kernel takes (scores and the other output columns are unchanged;
        # the softmax scale still comes from the true head dimension)
        dp = 64 if d < 64 else 128
        q3, k3, v3 = (torch.nn.functional.pad(t, (0, dp - d)) for t in (q3, k3, v3))
    q3, k3, v3 = q3.contiguous(), k3.contiguous(), v3.contiguous()
    out = torch.empty_like(q3)
    rc = _lib.load().hx_attention(q3.data_ptr(), k3.data_ptr(), v3.data_ptr(), out.data_ptr(), bh, m_dim, n_dim, dp, d,
                                  _DT[q.dtype], _stream_ptr(q.device))
    _lib.check(rc, "hx_attention")
    if dp != d:
        out = out[..., :d].contiguous()
    return out.view(q.shape)


attention_op = torch.library.custom_op("helion_amd::attention", mutates_args=())(_attention_impl)


@attention_op.register_fake
def _(q, k, v):
    return torch.empty_like(q, memory_format=torch.contiguous_format)


# ------------------------------------------------------------------------------ what the Python entry points call
def _caller(impl, op):
    def call(*args):
        return eager(impl, op, *args)
    return call


fp8_gemm_call = _caller(_fp8_gemm_impl, fp8_gemm_op)
fp8_attention_call = _caller(_fp8_attention_impl, fp8_attention_op)
moe_matmul_ogs_call = _caller(_moe_matmul_ogs_impl, moe_matmul_ogs_op)
moe_routing_call = _caller(_moe_routing_impl, moe_routing_op)
moe_matmul_topk_call = _caller(_moe_matmul_topk_impl, moe_matmul_topk_op)
cast_e4m3_x3_call = _caller(_cast_e4m3_x3_impl, cast_e4m3_x3_op)
fp8_quantize_call = _caller(_fp8_quantize_impl, fp8_quantize_op)
matmul_call = _caller(_matmul_impl, matmul_op)
attention_call = _caller(_attention_impl, attention_op)
