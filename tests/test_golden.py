"""The CPU oracle reproduces the committed fixtures bit for bit (guards the checker itself)."""
import pathlib

import numpy as np
import torch

from oracle import oracle as orc

G = pathlib.Path(__file__).resolve().parent / "golden"
E4M3 = torch.float8_e4m3fn


def _fp8(a):
    return torch.from_numpy(a.copy()).view(E4M3)


def test_gemm_fixture():
    z = np.load(G / "fp8_gemm_small.npz")
    for name in ("ragged", "skinny"):
        x, yt = _fp8(z[f"{name}_x"]), _fp8(z[f"{name}_yt"])
        sa, sb = (torch.tensor(float(s)) for s in z[f"{name}_scales"])
        got = orc.fp8_gemm(x, yt.T, sa, sb, torch.bfloat16).view(torch.int16).numpy()
        assert np.array_equal(got, z[f"{name}_out_bf16"])
        assert np.array_equal(orc.fp8_gemm(x, yt.T).view(torch.int16).numpy(), z[f"{name}_out_f16_unit"])


def test_attention_fixture():
    z = np.load(G / "fp8_attention_small.npz")
    for name in ("d64", "d128"):
        b, h, s, d = (int(v) for v in z[f"{name}_shape"])
        q, k, v = _fp8(z[f"{name}_q"]), _fp8(z[f"{name}_k"]), _fp8(z[f"{name}_v"])
        assert np.array_equal(orc.fp8_attention(q, k, v, b, h).view(torch.uint8).numpy(), z[f"{name}_out_e4m3"])
        assert np.array_equal(orc.fp8_attention(q, k, v, b, h, torch.float32).numpy(), z[f"{name}_out_f32"])


def test_moe_fixture():
    z = np.load(G / "moe_small.npz")
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        A = torch.from_numpy(z[f"{name}_A"].copy()).view(dt); W = torch.from_numpy(z[f"{name}_W"].copy()).view(dt)
        ex = torch.from_numpy(z[f"{name}_expert"].copy())
        got = orc.moe_matmul_ogs(*orc.moe_args_gen(A, W, ex)).view(torch.int16).numpy()
        assert np.array_equal(got, z[f"{name}_out"])


def test_siblings_fixture():
    z = np.load(G / "siblings_small.npz")
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        t = lambda key: torch.from_numpy(z[key].copy()).view(dt)
        x, y, bias = t(f"mm_{name}_x"), t(f"mm_{name}_y"), t(f"mm_{name}_bias")
        assert np.array_equal(orc.matmul(x, y).view(torch.int16).numpy(), z[f"mm_{name}_out"])
        assert np.array_equal(orc.matmul(x, y, bias, relu=True).view(torch.int16).numpy(), z[f"mm_{name}_out_bias_relu"])
        for tag in ("d64", "d128"):
            q, k, v = (t(f"att_{name}_{tag}_{c}") for c in "qkv")
            assert np.array_equal(orc.attention(q, k, v).view(torch.int16).numpy(), z[f"att_{name}_{tag}_out"])
