"""The C-ABI calls of helion_amd/ops.py made against the host execution model (tests/sim/libhx_sim.so) with operands in
guarded buffers: same arguments, same workspace queries, CPU tensors in place of device tensors.  Each function returns
the output tensor (a clone taken before the buffers are released)."""
from __future__ import annotations

import torch

from helion_amd import _lib as real

from . import simlib

_DT = {torch.float16: real.HX_F16, torch.bfloat16: real.HX_BF16, torch.float32: real.HX_F32, torch.float8_e4m3fn: real.HX_E4M3}
E4 = torch.float8_e4m3fn


def _p(t):
    return t.data_ptr() if t is not None else None


def fp8_gemm(x, y, scale_a=None, scale_b=None, out_dtype=torch.bfloat16, end_flush=True, want_path=None, lda=None, poison_ws=None,
             ws_after=None, ws_bytes=None, in_flight_of_b=False):
    """x [M,K] e4m3 (row-major), y [K,N] e4m3 with any of the two layouts the op passes on (strides kept).
    in_flight_of_b: simlib.work()'s in-flight figures count only the DMA that reads y."""
    lib = simlib.load()
    m, k = x.shape
    n = y.shape[1]
    with simlib.Arena(end_flush) as ar:
        if lda is None or lda == k:
            X, lda = ar.put(x), k
        else:  # rows padded to lda bytes
            buf = torch.zeros(m, lda, dtype=torch.uint8)
            buf[:, :k] = x.view(torch.uint8)
            X = ar.put(buf)
        if y.stride(1) == 1 or n == 1:  # row-major
            Y, ldb_k, ldb_n = ar.put(y.contiguous()), (n if k > 1 else 1), 1
            if n == 1:
                ldb_n = max(k, 1)
        else:  # column-major: memory is y^T [N,K]
            Y, ldb_k, ldb_n = ar.put(y.t().contiguous()), 1, k
        C = ar.out((m, n), out_dtype, fill=0xFF)
        sa = ar.put(scale_a.reshape(1).float()) if scale_a is not None else None
        sb = ar.put(scale_b.reshape(1).float()) if scale_b is not None else None
        if want_path is not None:
            got = lib.hx_fp8_gemm_path(m, n, k, lda, ldb_k, ldb_n, n, X.data_ptr(), Y.data_ptr(), C.data_ptr())
            assert got == want_path, f"fp8_gemm path {got}, expected {want_path}"
        wsb = lib.hx_fp8_gemm_workspace_bytes(m, n, k, ldb_k, ldb_n) if ws_bytes is None else ws_bytes
        ws = ar.empty(wsb) if wsb else None
        if ws is not None and poison_ws is not None:
            ws.copy_(poison_ws(wsb))
        if in_flight_of_b:
            lib.hx_sim_in_flight_source(Y.data_ptr(), Y.numel())
        rc = lib.hx_fp8_gemm(X.data_ptr(), Y.data_ptr(), C.data_ptr(), m, n, k, lda, ldb_k, ldb_n, n, _p(sa), _p(sb), _DT[out_dtype],
                             _p(ws), wsb, None)
        lib.hx_sim_in_flight_source(None, 0)
        simlib.check(rc, "hx_fp8_gemm")
        if ws_after is not None and ws is not None:
            ws_after.append(ws.clone())
        return C.clone()


def fp8_attention(q, k, v, batch, heads, out_dtype=E4, exact_max=True, v_layout="DS", end_flush=True, want_path=None, scale_dim=None):
    """q, k [BH,S,D]; v logically [BH,D,S], stored [D][S] ("DS") or [S][D] ("SD") per head."""
    lib = simlib.load()
    bh, s, d = q.shape
    with simlib.Arena(end_flush) as ar:
        Q, K = ar.put(q), ar.put(k)
        if v_layout == "SD":
            V, vsd, vss = ar.put(v.transpose(1, 2).contiguous()), 1, d
        else:
            V, vsd, vss = ar.put(v.contiguous()), s, 1
        O = ar.out((batch, heads, s, d), out_dtype, fill=0xFF)
        if want_path is not None:
            got = lib.hx_fp8_attention_path(bh, s, d, vsd, vss, Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr())
            assert got == want_path, f"fp8_attention path {got}, expected {want_path}"
        rc = lib.hx_fp8_attention(Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), bh, s, d, scale_dim or d, vsd, vss,
                                  _DT[out_dtype], int(exact_max), None)
        simlib.check(rc, "hx_fp8_attention")
        return O.clone()


def moe_grouped_gemm(A, W, counts, offsets, idx, static=False, end_flush=True, want_path=None, poison=None):
    lib = simlib.load()
    T, K = A.shape
    E, _, N = W.shape
    dt = A.dtype
    with simlib.Arena(end_flush) as ar:
        a, w = ar.put(A), ar.put(W)
        c = ar.out((T, N), dt, fill=0xFF)
        if poison is not None:
            c.fill_(poison)
        cn, of, ix = ar.put(counts.to(torch.int32)), ar.put(offsets.to(torch.int32)), ar.put(idx.to(torch.int32))
        if want_path is not None:
            got = lib.hx_moe_path(T, K, N, E, 1, a.data_ptr(), w.data_ptr(), c.data_ptr())
            assert got == want_path, f"moe path {got}, expected {want_path}"
        mt = int(counts.max()) if counts.numel() else 0
        if static:
            rc = lib.hx_moe_grouped_gemm_static(a.data_ptr(), w.data_ptr(), c.data_ptr(), cn.data_ptr(), of.data_ptr(), ix.data_ptr(),
                                                T, K, N, E, mt, _DT[dt], None)
            simlib.check(rc, "hx_moe_grouped_gemm_static")
        else:
            wsb = lib.hx_moe_workspace_bytes_shape(T, K, N, E)
            ws = ar.empty(wsb)
            ws.fill_(0xA5)
            rc = lib.hx_moe_grouped_gemm(a.data_ptr(), w.data_ptr(), c.data_ptr(), cn.data_ptr(), of.data_ptr(), ix.data_ptr(),
                                         T, K, N, E, mt, _DT[dt], ws.data_ptr(), wsb, None)
            simlib.check(rc, "hx_moe_grouped_gemm")
        return c.clone()


def moe_routing(ids, E, end_flush=True):
    lib = simlib.load()
    T = ids.numel()
    with simlib.Arena(end_flush) as ar:
        x = ar.put(ids)
        counts, offsets = ar.out((E,), torch.int32, fill=0xFF), ar.out((E + 1,), torch.int32, fill=0xFF)
        idx, mx = ar.out((T,), torch.int32, fill=0xFF), ar.out((1,), torch.int32, fill=0xFF)
        wsb = lib.hx_moe_routing_workspace_bytes(T, E)
        ws = ar.empty(wsb) if wsb else None
        if ws is not None:
            ws.fill_(0xA5)
        rc = lib.hx_moe_routing(x.data_ptr(), int(ids.dtype == torch.int64), T, E, counts.data_ptr(), offsets.data_ptr(), idx.data_ptr(),
                                mx.data_ptr(), _p(ws), wsb, None)
        simlib.check(rc, "hx_moe_routing")
        return counts.clone(), offsets.clone(), idx.clone(), mx.clone()


def moe_topk(A_tok, W, ids, top_k, end_flush=True):
    lib = simlib.load()
    T_tok, K = A_tok.shape
    E, _, N = W.shape
    dt = A_tok.dtype
    with simlib.Arena(end_flush) as ar:
        a, w, x = ar.put(A_tok), ar.put(W), ar.put(ids.reshape(-1))
        c = ar.out((T_tok * top_k, N), dt, fill=0xFF)
        wsb = lib.hx_moe_topk_workspace_bytes(T_tok, top_k, E)
        ws = ar.empty(wsb)
        ws.fill_(0xA5)
        rc = lib.hx_moe_topk_matmul(a.data_ptr(), w.data_ptr(), c.data_ptr(), x.data_ptr(), int(ids.dtype == torch.int64), T_tok, top_k,
                                    K, N, E, _DT[dt], ws.data_ptr(), wsb, None)
        simlib.check(rc, "hx_moe_topk_matmul")
        return c.clone()


def cast_e4m3_x3(q, k, v, end_flush=True):
    lib = simlib.load()
    with simlib.Arena(end_flush) as ar:
        ins = [ar.put(t) for t in (q, k, v)]
        outs = [ar.out(t.shape, E4, fill=0x7F) for t in (q, k, v)]
        rc = lib.hx_fp8_attention_preprocess(*[t.data_ptr() for t in ins], *[t.data_ptr() for t in outs], q.numel(), _DT[q.dtype], None)
        simlib.check(rc, "hx_fp8_attention_preprocess")
        return [t.clone() for t in outs]


def fp8_quantize(x, end_flush=True):
    lib = simlib.load()
    with simlib.Arena(end_flush) as ar:
        X = ar.put(x)
        Q = ar.out(x.shape, E4, fill=0x7F)
        scale = ar.out((1,), torch.float32, fill=0xFF)
        wsb = lib.hx_fp8_quantize_workspace_bytes(x.numel())
        ws = ar.empty(wsb)
        ws.fill_(0xA5)
        rc = lib.hx_fp8_quantize(X.data_ptr(), Q.data_ptr(), x.numel(), _DT[x.dtype], scale.data_ptr(), ws.data_ptr(), wsb, None)
        simlib.check(rc, "hx_fp8_quantize")
        return Q.clone(), scale.clone()[0]


def matmul(x, y, bias=None, relu=False, out_dtype=None, split_k=1, end_flush=True, want_path=None, want_splits=None):
    lib = simlib.load()
    m, k = x.shape
    n = y.shape[1]
    dt = x.dtype
    out_dtype = out_dtype or dt
    with simlib.Arena(end_flush) as ar:
        X = ar.put(x)
        if y.stride(1) == 1 or n == 1:
            Y, ldb_k, ldb_n = ar.put(y.contiguous()), n, 1
        else:
            Y, ldb_k, ldb_n = ar.put(y.t().contiguous()), 1, k
        B = ar.put(bias) if bias is not None else None
        C = ar.out((m, n), out_dtype, fill=0xFF)
        has_ep = int(bias is not None or relu)
        if want_path is not None:
            got = lib.hx_matmul_path(m, n, k, k, ldb_k, ldb_n, n, _DT[dt], X.data_ptr(), Y.data_ptr(), C.data_ptr(), _p(B))
            assert got == want_path, f"matmul path {got}, expected {want_path}"
        if want_splits is not None:
            got = lib.hx_matmul_splits(m, n, k, k, ldb_k, ldb_n, n, _DT[dt], split_k)
            assert got == want_splits, f"matmul splits {got}, expected {want_splits}"
        wsb = lib.hx_matmul_workspace_bytes(m, n, k, k, ldb_k, ldb_n, n, _DT[dt], _DT[out_dtype], has_ep, split_k)
        ws = ar.empty(wsb) if wsb else None
        if ws is not None:
            ws.fill_(0xFF)
        rc = lib.hx_matmul(X.data_ptr(), Y.data_ptr(), C.data_ptr(), m, n, k, k, ldb_k, ldb_n, n, _p(B), _DT[bias.dtype] if bias is not None else 0,
                           int(relu), _DT[dt], _DT[out_dtype], split_k, _p(ws), wsb, None)
        simlib.check(rc, "hx_matmul")
        return C.clone()


def attention16(q, k, v, scale_dim=None, end_flush=True, want_path=None):
    """q [BH,M,D], k, v [BH,N,D] contiguous, one dtype."""
    lib = simlib.load()
    bh, m, d = q.shape
    n = k.shape[1]
    with simlib.Arena(end_flush) as ar:
        Q, K, V = ar.put(q), ar.put(k), ar.put(v)
        O = ar.out(q.shape, q.dtype, fill=0xFF)
        if want_path is not None:
            got = lib.hx_attention_path(bh, m, n, d, _DT[q.dtype], Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr())
            assert got == want_path, f"attention path {got}, expected {want_path}"
        rc = lib.hx_attention(Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), bh, m, n, d, scale_dim or d, _DT[q.dtype], None)
        simlib.check(rc, "hx_attention")
        return O.clone()
