"""Drop-in for the reference's examples/fp8_gemm.py: same callables, same signatures, same layouts and
output dtype, backed by the gfx950 HIP kernels."""
from __future__ import annotations

import torch

from .ops import fp8_gemm_call, fp8_quantize_call


def fp8_gemm(x: torch.Tensor, y: torch.Tensor, *, scale_a: torch.Tensor | None = None,
             scale_b: torch.Tensor | None = None, out_dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """``out[m,n] = fp16(sum_k x[m,k] * y[k,n])`` with fp32 accumulation (reference:
    examples/fp8_gemm.py:29-57).  x: [m,k] float8_e4m3fn, y: [k,n] float8_e4m3fn with any strides
    (column-major y, strides (1,k), is the fast layout).  Keyword-only extensions, all defaulting to
    the reference behaviour: per-tensor fp32 scales (one-element device tensors) and ``out_dtype``."""
    return fp8_gemm_call(x, y, scale_a, scale_b, out_dtype)


def fp8_gemm_scaled(x: torch.Tensor, y: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                    out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``cast((x @ y) * scale_a * scale_b)`` — the per-tensor-scaled form torch._scaled_mm computes."""
    return fp8_gemm_call(x, y, scale_a, scale_b, out_dtype)


def fp8_quantize_per_tensor(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-tensor e4m3 quantisation for ``fp8_gemm_scaled``: returns ``(q, scale)`` with ``scale = max|x| / 448``
    (1 for an all-zero tensor) and ``q = (x * (448 / max|x|)).to(float8_e4m3fn)``, so ``q.float() * scale ~ x``.
    Three launches, no host synchronisation.  (The reference's example only ever passes unit scales,
    examples/fp8_gemm.py:74-78; this is the producer of real ones.)"""
    return fp8_quantize_call(x)


def reference_fp8_gemm_pytorch(x_fp8: torch.Tensor, y_fp8: torch.Tensor) -> torch.Tensor:
    """The reference's baseline (examples/fp8_gemm.py:61-78): torch._scaled_mm with unit scales, fp16 out."""
    y_fp8_t = y_fp8.T.contiguous().T
    scale_a = torch.tensor(1.0, device=x_fp8.device)
    scale_b = torch.tensor(1.0, device=x_fp8.device)
    return torch._scaled_mm(x_fp8, y_fp8_t, scale_a, scale_b, use_fast_accum=False, out_dtype=torch.float16)


def fp8_gemm_tritonbench(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """examples/fp8_gemm.py:82-91."""
    return fp8_gemm(a, b)


def check(m: int, k: int, n: int) -> None:
    """examples/fp8_gemm.py:95-109: randn -> e4m3 operands (row-major y), kernel against torch._scaled_mm."""
    from .testing import run_example

    x = torch.randn([m, k], device="cuda", dtype=torch.float32).to(torch.float8_e4m3fn)
    y = torch.randn([k, n], device="cuda", dtype=torch.float32).to(torch.float8_e4m3fn)
    run_example(fp8_gemm, reference_fp8_gemm_pytorch, (x, y))


def main() -> None:
    """examples/fp8_gemm.py:113-119."""
    check(256, 256, 256)
    check(512, 512, 512)
    check(1024, 1024, 1024)


if __name__ == "__main__":
    main()
