"""Writes the small golden fixtures in this directory from the pinned CPU oracle (oracle/oracle.py).

The reference ships no numeric vectors for these kernels (its tests compare against eager PyTorch at
run time), so the fixtures freeze the oracle's outputs on seeded inputs: they guard the oracle against
silent change (tests/test_golden.py, CPU) and give the GPU tests a file-based anchor that does not
depend on the oracle code at all.  Inputs and outputs are stored as raw integer codes.

    python tests/golden/make_golden.py
"""
import pathlib
import sys

import numpy as np
import torch

ROOT = pathlib.Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import oracle as orc  # noqa: E402

HERE = pathlib.Path(__file__).resolve().parent
E4M3 = torch.float8_e4m3fn


def u8(t):
    return t.contiguous().view(torch.uint8).numpy()


def i16(t):
    return t.contiguous().view(torch.int16).numpy()


def siblings(g):
    """16-bit siblings: matmul 96x64x72 with bias and relu, attention M=80 N=100 D=64 (ragged) and M=N=64 D=128, one head each."""
    out = {}
    for name, dt in {"bf16": torch.bfloat16, "f16": torch.float16}.items():
        x = torch.randn(96, 64, generator=g).to(dt); y = torch.randn(64, 72, generator=g).to(dt)
        bias = torch.randn(72, generator=g).to(dt)
        out[f"mm_{name}_x"] = i16(x); out[f"mm_{name}_y"] = i16(y); out[f"mm_{name}_bias"] = i16(bias)
        out[f"mm_{name}_out"] = i16(orc.matmul(x, y))
        out[f"mm_{name}_out_bias_relu"] = i16(orc.matmul(x, y, bias, relu=True))
        for tag, (bh, m, n, d) in {"d64": (1, 80, 100, 64), "d128": (1, 64, 64, 128)}.items():
            q = torch.randn(bh, m, d, generator=g).to(dt); k = torch.randn(bh, n, d, generator=g).to(dt)
            v = torch.randn(bh, n, d, generator=g).to(dt)
            out[f"att_{name}_{tag}_q"] = i16(q); out[f"att_{name}_{tag}_k"] = i16(k); out[f"att_{name}_{tag}_v"] = i16(v)
            out[f"att_{name}_{tag}_out"] = i16(orc.attention(q, k, v))
    np.savez_compressed(HERE / "siblings_small.npz", **out)


def main():
    g = torch.Generator().manual_seed(1234)
    # fp8 gemm: 48x40x96 (ragged, general kernel) and 16x64x256 (skinny) with scales
    out = {}
    for name, (m, n, k) in {"ragged": (48, 40, 96), "skinny": (16, 64, 256)}.items():
        x = torch.randn(m, k, generator=g).clamp(-448, 448).to(E4M3)
        yt = torch.randn(n, k, generator=g).clamp(-448, 448).to(E4M3)
        sa, sb = torch.tensor(1.25), torch.tensor(0.75)
        out[f"{name}_x"] = u8(x); out[f"{name}_yt"] = u8(yt)
        out[f"{name}_scales"] = np.array([1.25, 0.75], dtype=np.float32)
        out[f"{name}_out_bf16"] = i16(orc.fp8_gemm(x, yt.T, sa, sb, torch.bfloat16))
        out[f"{name}_out_f16_unit"] = i16(orc.fp8_gemm(x, yt.T))
    np.savez_compressed(HERE / "fp8_gemm_small.npz", **out)

    # fp8 attention: B1 H2 S64 D64 and B1 H1 S128 D128
    out = {}
    for name, (b, h, s, d) in {"d64": (1, 2, 64, 64), "d128": (1, 1, 128, 128)}.items():
        q, k, v = (torch.randn(b, h, s, d, generator=g) for _ in range(3))
        q8, k8, v8 = orc.preprocess_fp8_attention_inputs(q, k, v)
        out[f"{name}_q"] = u8(q8); out[f"{name}_k"] = u8(k8); out[f"{name}_v"] = u8(v8)
        out[f"{name}_shape"] = np.array([b, h, s, d])
        out[f"{name}_out_e4m3"] = u8(orc.fp8_attention(q8, k8, v8, b, h))
        out[f"{name}_out_f32"] = orc.fp8_attention(q8, k8, v8, b, h, torch.float32).numpy()
    np.savez_compressed(HERE / "fp8_attention_small.npz", **out)

    # moe: T=96 K=64 N=48 E=5 (expert 3 empty), bf16 and fp16
    out = {}
    for name, dt in {"bf16": torch.bfloat16, "f16": torch.float16}.items():
        A = torch.randn(96, 64, generator=g).to(dt); W = (torch.randn(5, 64, 48, generator=g) * 0.1).to(dt)
        ex = torch.randint(5, (96,), generator=g); ex[ex == 3] = 0
        out[f"{name}_A"] = i16(A); out[f"{name}_W"] = i16(W); out[f"{name}_expert"] = ex.numpy().astype(np.int64)
        out[f"{name}_out"] = i16(orc.moe_matmul_ogs(*orc.moe_args_gen(A, W, ex)))
    np.savez_compressed(HERE / "moe_small.npz", **out)
    siblings(torch.Generator().manual_seed(4321))
    for f in sorted(HERE.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
