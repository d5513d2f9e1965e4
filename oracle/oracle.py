"""CPU oracle: a restatement of Helion's *ref-eager* execution of the three example kernels.

TEST INFRASTRUCTURE ONLY.  Nothing under ``helion_amd/`` imports this module; it is used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` as
the checker / the timed CPU reference, never as the product path.

What it restates (paths relative to the reference checkout):

* ``examples/fp8_gemm.py:29-57``           -> :func:`fp8_gemm`
* ``helion/language/matmul_ops.py:214-249`` -> :func:`hl_dot_fp8` (``torch._scaled_mm`` with unit
  scales, ``out_dtype`` = accumulator dtype, then ``acc + result``)
* ``examples/fp8_attention.py:22-106``     -> :func:`fp8_attention`
* ``examples/moe_matmul_ogs.py:84-148``    -> :func:`moe_args_gen`, :func:`moe_matmul_ogs`
* ``examples/matmul.py:25-56``, ``examples/matmul_split_k.py:30-68`` -> :func:`matmul`
* ``examples/attention.py:33-84``          -> :func:`attention`
* ``helion/language/loops.py:491-533``     -> "one tile spans the whole dimension" in ref mode,
  which is why every tiled loop below has exactly one iteration.

Pinning status (see tests/test_oracle_*.py):

* e4m3 decode/encode tables : closed form vs ``torch.float8_e4m3fn`` casts over all 256 codes and
  all rounding midpoints; C restatement in ``oracle/ref_c.c`` agrees bit for bit.
* fp8_gemm                  : float64 brute force on small shapes; bit-equality with CPU
  ``torch._scaled_mm`` (the routine the reference calls) after fp16/bf16 rounding.
* fp8_attention             : float64 brute force (S<=32), closed-form special cases (S=1,
  uniform scores), permutation invariance, row-max-of-p == 1, a statement-by-statement walk of the
  reference kernel body with a single tile.
* fp8_attention_tiled       : the same reference lines with the key loop in tiles (the compiled kernel's online
  softmax); equals fp8_attention for one tile, float64 re-derivation with explicit loops, tile-size invariance
  where p is exactly representable.
* fp8_quantize_per_tensor   : the reference has no such function (it only ever passes unit scales,
  ``examples/fp8_gemm.py:74-78``), so there is nothing of the reference's to pin it against: it is the
  build's own definition (amax / 448 scaling), pinned by its algebraic properties (exact powers of two,
  the amax element lands on +-448, dequantisation error within half an e4m3 step) and by the numpy
  e4m3 encoder above.
* matmul (16-bit / fp32, bias and relu epilogues, also the split-K example, whose eager mode has
  one split): float64 brute force on small shapes, identity-matrix and zero-operand special cases,
  the relation the reference's tests assert (``x @ y``, ``relu(x @ y + bias)``:
  ``test/test_examples.py:33-46,143-200,460-474``).
* attention (16-bit / fp32): float64 brute force with explicit loops, closed-form special cases
  (one key, uniform scores, a dominant key), key-permutation invariance, and the relation the
  reference's tests assert (``scaled_dot_product_attention``: ``test/test_examples.py:342-390``).
* moe_matmul_ogs            : the reference's own unit test skips the accuracy check
  (``test/test_examples.py:434-458``), so the *reference's tests* pin nothing here; the oracle is
  pinned by the semantic definition ``moe_matmul_ogs_reference`` (per-expert dense matmul),
  invariants of the routing tables and float64 brute force.
"""
from __future__ import annotations

import math

import numpy as np
import torch

# --------------------------------------------------------------------------------------
# OCP float8 e4m3fn, closed form (no torch involved): sign(1) exp(4, bias 7) mantissa(3);
# exp==0 -> subnormal m/8 * 2^-6; 0x7f / 0xff are NaN; there is no infinity.
# --------------------------------------------------------------------------------------


def _build_decode_table() -> np.ndarray:
    t = np.empty(256, dtype=np.float32)
    for code in range(256):
        s, e, m = code >> 7, (code >> 3) & 0xF, code & 7
        if e == 0xF and m == 7:
            v = float("nan")
        elif e == 0:
            v = (m / 8.0) * 2.0**-6
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[code] = -v if s else v
    return t


E4M3_DECODE_TABLE = _build_decode_table()
_POS_VALUES = E4M3_DECODE_TABLE[:0x7F].astype(np.float64)  # 0 .. 448, ascending


def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    """uint8 codes -> float32 values (exact)."""
    return E4M3_DECODE_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> uint8 e4m3fn codes, round-to-nearest-even, torch semantics:
    |x| <= 464 rounds (saturating at 448), |x| > 464 and NaN give the NaN code."""
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    hi = np.searchsorted(_POS_VALUES, a, side="left")  # first value >= a
    hi = np.clip(hi, 0, len(_POS_VALUES) - 1)
    lo = np.clip(hi - 1, 0, len(_POS_VALUES) - 1)
    dlo = np.abs(a - _POS_VALUES[lo])
    dhi = np.abs(_POS_VALUES[hi] - a)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(a > 464.0, 0x7F, code).astype(np.uint8)
    code = np.where(np.isnan(x), 0x7F, code).astype(np.uint8)
    sign = (np.signbit(x).astype(np.uint8)) << 7
    return (code | sign).astype(np.uint8)


def dq(t: torch.Tensor) -> torch.Tensor:
    """e4m3fn tensor -> float32 (exact), through the closed-form table."""
    codes = t.contiguous().view(torch.uint8).numpy()
    return torch.from_numpy(e4m3_decode(codes)).reshape(t.shape)


def to_e4m3(t: torch.Tensor) -> torch.Tensor:
    """float32 tensor -> float8_e4m3fn through the closed-form encoder."""
    codes = e4m3_encode(t.contiguous().numpy())
    return torch.from_numpy(codes).view(torch.float8_e4m3fn).reshape(t.shape)


# --------------------------------------------------------------------------------------
# fp8_gemm
# --------------------------------------------------------------------------------------


def hl_dot_fp8(mat1: torch.Tensor, mat2: torch.Tensor, acc: torch.Tensor | None = None) -> torch.Tensor:
    """helion/language/matmul_ops.py:214-249 — the literal ref-mode ``hl.dot`` for fp8 operands."""
    out_dtype = torch.float32 if acc is None else acc.dtype
    mat2_t = mat2.T.contiguous().T
    one = torch.tensor(1.0)
    result = torch._scaled_mm(mat1, mat2_t, one, one, use_fast_accum=False, out_dtype=out_dtype)
    return result if acc is None else acc + result


def fp8_gemm_ref_eager(x: torch.Tensor, y: torch.Tensor, out_dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """examples/fp8_gemm.py:42-57 walked with one tile per loop (this is what is timed as the CPU
    baseline: ATen's CPU ``_scaled_mm``)."""
    m, k = x.shape
    k2, n = y.shape
    assert k == k2, f"size mismatch {k} != {k2}"
    acc = torch.zeros(m, n, dtype=torch.float32)
    acc = hl_dot_fp8(x, y, acc=acc)
    return acc.to(out_dtype)


def fp8_gemm(
    x: torch.Tensor,
    y: torch.Tensor,
    scale_a: float | torch.Tensor = 1.0,
    scale_b: float | torch.Tensor = 1.0,
    out_dtype: torch.dtype = torch.float16,
) -> torch.Tensor:
    """Closed form of the above: fp32(x) @ fp32(y) accumulated in fp32, times the fp32 product
    ``scale_a*scale_b`` (an extension; the reference hard-codes 1.0, examples/fp8_gemm.py:74-75),
    rounded once to ``out_dtype``."""
    acc = dq(x) @ dq(y)
    alpha = torch.as_tensor(scale_a, dtype=torch.float32) * torch.as_tensor(scale_b, dtype=torch.float32)
    return (acc * alpha).to(out_dtype)


# --------------------------------------------------------------------------------------
# fp8_attention
# --------------------------------------------------------------------------------------


def attention_scale(head_dim: int) -> torch.Tensor:
    """examples/fp8_attention.py:50-52: python-double ``1/sqrt(D) * 1.44269504``; it becomes fp32
    when it multiplies the fp32 score tensor (test/test_examples.expected:742-743 shows the fp32
    literal 0.18033688 for D=64)."""
    return torch.tensor((1.0 / math.sqrt(float(head_dim))) * 1.44269504, dtype=torch.float32)


def fp8_attention(
    q: torch.Tensor,  # [BH, S, D] e4m3
    k: torch.Tensor,  # [BH, S, D] e4m3
    v: torch.Tensor,  # [BH, D, S] e4m3 (pre-transposed)
    batch: int,
    heads: int,
    out_dtype: torch.dtype = torch.float8_e4m3fn,
) -> torch.Tensor:
    """examples/fp8_attention.py:42-106 with every ``hl.tile`` covering its whole dimension, so
    the row max is the exact row max, ``alpha`` multiplies zeros, and the un-normalised ``p`` is
    cast to e4m3 relative to that exact max; ``l`` sums the un-quantised p."""
    bh, s, d = q.shape
    assert bh == batch * heads
    c = attention_scale(d)
    out = torch.empty(batch, heads, s, d, dtype=out_dtype)
    for i in range(bh):
        qk = dq(q[i]) @ dq(k[i]).T  # fp32, exact products, fp32 sums
        qk_scaled = qk * c
        m = torch.amax(qk_scaled, dim=-1)
        p = torch.exp2(qk_scaled - m[:, None])
        l = torch.sum(p, dim=-1)
        p8 = to_e4m3(p)
        acc = dq(p8) @ dq(v[i]).T
        acc = acc / l[:, None]
        out[i // heads, i % heads] = acc.to(out_dtype)
    return out


def fp8_attention_literal(q, k, v, batch, heads):
    """Statement-by-statement walk of examples/fp8_attention.py:54-105 (single tile per loop),
    including the -inf / alpha first-iteration path, using the literal ref-mode ``hl.dot``.
    Used only to pin :func:`fp8_attention`."""
    bh, s, d = q.shape
    out = torch.empty(batch, heads, s, d, dtype=torch.float8_e4m3fn)
    sm_scale = 1.0 / math.sqrt(float(d))
    sm_scale = sm_scale * 1.44269504
    for i in range(bh):
        b, h = i // heads, i % heads
        m_i = torch.full([s], float("-inf"), dtype=torch.float32)
        l_i = torch.full([s], 0.0, dtype=torch.float32)
        acc = torch.zeros([s, d], dtype=torch.float32)
        q_tile = q[i]
        k_tile_t = k[i].transpose(0, 1)
        qk = hl_dot_fp8(q_tile, k_tile_t)
        qk_scaled = qk * sm_scale
        qk_max = torch.amax(qk_scaled, dim=-1)
        m_new = torch.maximum(m_i, qk_max)
        qk_shifted = qk_scaled - m_new[:, None]
        p = torch.exp2(qk_shifted)
        l_ij = torch.sum(p, dim=-1)
        alpha = torch.exp2(m_i - m_new)
        l_i = l_i * alpha + l_ij
        acc = acc * alpha[:, None]
        v_tile = v[i]
        p_fp8 = p.to(v.dtype)
        acc = hl_dot_fp8(p_fp8, v_tile.t(), acc=acc)
        acc = acc / l_i[:, None]
        out[b, h] = acc.to(torch.float8_e4m3fn)
    return out


def fp8_attention_tiled(q, k, v, batch, heads, tile_n: int, out_dtype: torch.dtype = torch.float8_e4m3fn):
    """examples/fp8_attention.py:54-105 with the key loop (``for tile_n in hl.tile(seq_len)``, :66) walked in tiles of
    ``tile_n`` keys instead of one tile for the whole sequence: the online-softmax form the reference's compiled
    kernel executes (its tile size is an autotuned config value; ref-eager mode is the ``tile_n >= seq_len`` case and
    then this function equals :func:`fp8_attention` bit for bit).  Each statement of the loop body is restated in
    order: scores of the tile, running max, p against the running max, l and acc rescaled by alpha, p cast to e4m3
    for the second product.  The query tile spans the whole sequence (rows are independent of one another).
    Pinned by: equality with :func:`fp8_attention` for one tile; an independent float64 re-derivation in
    tests/test_oracle_attention.py (explicit per-row loops, own e4m3 rounding through the numpy encoder); invariance
    of the result to tile_n when every p is exactly representable (uniform scores)."""
    bh, s, d = q.shape
    assert bh == batch * heads
    c = attention_scale(d)
    out = torch.empty(batch, heads, s, d, dtype=out_dtype)
    for i in range(bh):
        m_i = torch.full([s], float("-inf"), dtype=torch.float32)
        l_i = torch.zeros([s], dtype=torch.float32)
        acc = torch.zeros([s, d], dtype=torch.float32)
        qf, kf, vf = dq(q[i]), dq(k[i]), dq(v[i])
        for n0 in range(0, s, tile_n):
            n1 = min(n0 + tile_n, s)
            qk_scaled = (qf @ kf[n0:n1].T) * c
            m_new = torch.maximum(m_i, torch.amax(qk_scaled, dim=-1))
            p = torch.exp2(qk_scaled - m_new[:, None])
            l_ij = torch.sum(p, dim=-1)
            alpha = torch.exp2(m_i - m_new)
            l_i = l_i * alpha + l_ij
            acc = acc * alpha[:, None]
            acc = acc + dq(to_e4m3(p)) @ vf[:, n0:n1].T
            m_i = m_new
        out[i // heads, i % heads] = (acc / l_i[:, None]).to(out_dtype)
    return out


def preprocess_fp8_attention_inputs(q, k, v):
    """examples/fp8_attention.py:110-133."""
    q8 = q.to(torch.float8_e4m3fn)
    k8 = k.to(torch.float8_e4m3fn)
    v8 = v.permute(0, 1, 3, 2).to(torch.float8_e4m3fn)
    b, h, s, d = q.shape
    return q8.reshape(b * h, s, d), k8.reshape(b * h, s, d), v8.reshape(b * h, d, s)


# --------------------------------------------------------------------------------------
# moe_matmul_ogs
# --------------------------------------------------------------------------------------


def fp8_quantize_per_tensor(x: torch.Tensor):
    """Definition of the per-tensor quantiser in front of the scaled GEMM (no counterpart in the reference):
    ``amax = max|x|`` in fp32; ``scale = amax / 448`` (1 if amax == 0); ``q = e4m3(x * (448 / amax))`` with both
    divisions and the product rounded once in fp32.  Returns ``(q, scale)`` with ``scale`` a 0-d fp32 tensor."""
    xf = x.to(torch.float32)
    amax = xf.abs().max() if xf.numel() else torch.zeros((), dtype=torch.float32)
    if float(amax) == 0.0:
        return to_e4m3(xf), torch.ones((), dtype=torch.float32)
    c448 = torch.tensor(448.0, dtype=torch.float32)
    scale = amax / c448
    inv = c448 / amax
    return to_e4m3(xf * inv), scale


def moe_args_gen(A: torch.Tensor, W: torch.Tensor, expert_per_row: torch.Tensor):
    """examples/moe_matmul_ogs.py:84-121."""
    E = W.size(0)
    idx = torch.argsort(expert_per_row, stable=True).to(torch.int32)
    counts = torch.bincount(expert_per_row, minlength=E).to(torch.int32)
    offsets = torch.empty(E + 1, dtype=torch.int32)
    offsets[0] = 0
    offsets[1:] = torch.cumsum(counts, 0, dtype=torch.int32)
    max_t = int(counts.max().item())
    return A, W, counts, offsets, idx, torch.empty(max_t)


def moe_matmul_ogs(A, W, counts, offsets, idx, max_t_tensor=None) -> torch.Tensor:
    """Semantics of examples/moe_matmul_ogs.py:25-80 == moe_matmul_ogs_reference (:125-148):
    rows routed to expert e get A[rows] @ W[e], fp32 accumulation, one rounding to the promoted
    dtype; rows routed nowhere stay zero (C is zero-initialised, :49-54).  The reference kernel's
    read-modify-write of padded lanes (:75-79) is a race, not semantics, and is not restated."""
    T, K = A.shape
    E, _, N = W.shape
    dtype = torch.promote_types(A.dtype, W.dtype)
    C = torch.zeros(T, N, dtype=dtype)
    for e in range(E):
        n = int(counts[e])
        if n == 0:
            continue
        start = int(offsets[e])
        rows = idx[start : start + n].long()
        C[rows] = (A[rows].float() @ W[e].float()).to(dtype)
    return C


def moe_matmul_ogs_reference(A, W, expert_per_row) -> torch.Tensor:
    """examples/moe_matmul_ogs.py:125-148 computed with fp32 accumulation."""
    T, K = A.shape
    N = W.size(2)
    dtype = torch.promote_types(A.dtype, W.dtype)
    C = torch.zeros(T, N, dtype=dtype)
    for e in range(W.size(0)):
        rows = (expert_per_row == e).nonzero(as_tuple=True)[0]
        if rows.numel() == 0:
            continue
        C[rows] = (A[rows].float() @ W[e].float()).to(dtype)
    return C


# --------------------------------------------------------------------------------------------
# dense matmul with an epilogue (examples/matmul.py:25-56; examples/matmul_split_k.py:30-68 in eager mode, where the
# K dimension is one tile and therefore one split)
# --------------------------------------------------------------------------------------------
def matmul(x: torch.Tensor, y: torch.Tensor, bias: torch.Tensor | None = None, relu: bool = False,
           out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``acc = zeros(fp32); acc = addmm(acc, x, y)`` (examples/matmul.py:51-54; with an fp32 accumulator the eager mode
    computes ``mm(x, y, out_dtype=fp32) + acc``, helion/runtime/ref_mode.py:186-211: exact products, fp32 sums),
    ``out = epilogue(acc, tile)`` cast to ``promote_types(x.dtype, y.dtype)`` on the store (:55).  The epilogues
    restated are the ones the reference's examples and tests pass: ``acc + bias[tile[1]]`` (bias promoted to fp32 by
    the addition) and ``relu`` of it."""
    dt = torch.promote_types(x.dtype, y.dtype)
    acc = x.to(torch.float32) @ y.to(torch.float32)
    if bias is not None:
        acc = acc + bias.reshape(-1).to(torch.float32)
    if relu:
        acc = torch.relu(acc)
    return acc.to(out_dtype if out_dtype is not None else dt)


# --------------------------------------------------------------------------------------------
# 16-bit / fp32 attention (examples/attention.py:33-84)
# --------------------------------------------------------------------------------------------
def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """One key tile (the eager mode's ``hl.tile`` spans the whole key dimension, helion/language/loops.py:506-510), so
    the running max is the exact row max and the rescaling factor of the first and only step multiplies zeros:
    ``qk = q @ k^T`` (:64), ``m = amax(qk) * qk_scale`` (:65), ``p = exp2(qk * qk_scale - m)`` (:66-67),
    ``l = sum(p)`` (:68-70), ``acc = p.to(v.dtype) @ v`` in fp32 (:73-75), ``out = (acc / l).to(q.dtype)`` (:78-79).
    The scores are kept in fp32 here, as the compiled kernel's dot product does; the eager mode's ``torch.bmm`` of
    16-bit operands returns 16-bit scores, one more rounding that the tolerance of the parity tests covers."""
    d = q.shape[-1]
    qk_scale = (1.0 / math.sqrt(d)) * 1.44269504
    q3 = q.reshape(-1, q.shape[-2], d).to(torch.float32)
    k3 = k.reshape(-1, k.shape[-2], d).to(torch.float32)
    v3 = v.reshape(-1, v.shape[-2], d)
    qk = torch.bmm(q3, k3.transpose(1, 2))
    m = torch.amax(qk, -1) * qk_scale
    p = torch.exp2(qk * qk_scale - m[:, :, None])
    l = p.sum(-1)
    acc = torch.bmm(p.to(v.dtype).to(torch.float32), v3.to(torch.float32))
    return (acc / l[:, :, None]).to(q.dtype).view(q.shape)
