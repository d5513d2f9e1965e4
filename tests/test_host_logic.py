"""Host-side mirror of the reference's Python entry points: signatures, routing prep, preprocessing,
shape inference of the registered ops, and loud failure off-GPU."""
import inspect

import pytest
import torch

import helion_amd as hx
from oracle import oracle as orc


def test_signatures_match_the_reference_entry_points():
    # examples/fp8_gemm.py:30, examples/fp8_attention.py:23-29, examples/moe_matmul_ogs.py:26-33
    assert list(inspect.signature(hx.fp8_gemm).parameters)[:2] == ["x", "y"]
    assert list(inspect.signature(hx.fp8_attention_kernel).parameters)[:5] == ["q", "k", "v", "batch", "heads"]
    assert list(inspect.signature(hx.moe_matmul_ogs).parameters) == [
        "A", "W", "expert_token_counts", "expert_token_offsets", "sorted_to_orig_token_idx", "max_T_per_expert_tensor"]
    for name, p in inspect.signature(hx.fp8_gemm).parameters.items():
        if name not in ("x", "y"):
            assert p.kind is inspect.Parameter.KEYWORD_ONLY
    assert inspect.signature(hx.fp8_gemm).parameters["out_dtype"].default is torch.float16
    assert inspect.signature(hx.fp8_attention_kernel).parameters["out_dtype"].default is torch.float8_e4m3fn


def test_args_gen_matches_oracle_on_cpu():
    g = torch.Generator().manual_seed(0)
    A = torch.randn(64, 8, generator=g).half(); W = torch.randn(5, 8, 8, generator=g).half()
    ex = torch.randint(5, (64,), generator=g)
    ours = hx.moe_matmul_ogs_helion_kernel_args_gen(A, W, ex)
    ref = orc.moe_args_gen(A, W, ex)
    for a, b in zip(ours[2:5], ref[2:5]):
        assert torch.equal(a, b)
    assert ours[5].numel() == ref[5].numel()


def test_preprocess_matches_oracle_on_cpu():
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(2, 3, 16, 8, generator=g) for _ in range(3))
    for a, b in zip(hx.preprocess_fp8_attention_inputs(q, k, v), orc.preprocess_fp8_attention_inputs(q, k, v)):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert hx.preprocess_fp8_attention_inputs(q, k, v)[2].shape == (6, 8, 16)


def test_ops_refuse_cpu_tensors():
    x = torch.zeros(4, 4).to(torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="GPU only"):
        hx.fp8_gemm(x, x)
    with pytest.raises(RuntimeError, match="GPU only"):
        hx.fp8_attention_kernel(x.reshape(1, 4, 4), x.reshape(1, 4, 4), x.reshape(1, 4, 4), 1, 1)
    with pytest.raises(RuntimeError, match="GPU only"):
        hx.moe_matmul_ogs(torch.zeros(4, 4).half(), torch.zeros(1, 4, 4).half(), torch.zeros(1, dtype=torch.int32),
                          torch.zeros(2, dtype=torch.int32), torch.zeros(4, dtype=torch.int32), torch.empty(4))


def test_sibling_ops_refuse_cpu_tensors_and_epilogue_objects_are_plain_callables():
    from helion_amd.matmul import bias_add, bias_relu, relu
    x = torch.zeros(4, 4).half()
    with pytest.raises(RuntimeError, match="GPU only"):
        hx.matmul(x, x)
    with pytest.raises(RuntimeError, match="GPU only"):
        hx.attention(x.reshape(1, 4, 4), x.reshape(1, 4, 4), x.reshape(1, 4, 4))
    # the fused epilogues keep the reference's (acc, tile) calling convention (examples/matmul.py:30-34), so they can be
    # handed to any matmul that takes such a callable
    acc = torch.tensor([[-1.0, 2.0, 3.0]]); bias = torch.tensor([0.5, -4.0, 1.0]).half()
    tile = (slice(0, 1), slice(0, 3))
    assert torch.equal(bias_add(bias)(acc, tile), acc + bias.float())
    assert torch.equal(bias_relu(bias)(acc, tile), torch.relu(acc + bias.float()))
    assert torch.equal(bias_relu(bias.reshape(1, 3))(acc, tile), torch.relu(acc + bias.float()))
    assert torch.equal(relu()(acc, tile), torch.relu(acc))


def test_registered_ops_infer_shapes_on_meta_tensors():
    x = torch.empty(32, 64, dtype=torch.float8_e4m3fn, device="meta")
    y = torch.empty(64, 48, dtype=torch.float8_e4m3fn, device="meta")
    out = torch.ops.helion_amd.fp8_gemm(x, y, None, None, torch.float16)
    assert out.shape == (32, 48) and out.dtype == torch.float16
    q = torch.empty(6, 128, 64, dtype=torch.float8_e4m3fn, device="meta")
    v = torch.empty(6, 64, 128, dtype=torch.float8_e4m3fn, device="meta")
    o = torch.ops.helion_amd.fp8_attention(q, q, v, 2, 3, torch.float8_e4m3fn, True)
    assert o.shape == (2, 3, 128, 64) and o.dtype == torch.float8_e4m3fn
    A = torch.empty(10, 8, dtype=torch.bfloat16, device="meta"); W = torch.empty(3, 8, 12, dtype=torch.bfloat16, device="meta")
    i32 = lambda n: torch.empty(n, dtype=torch.int32, device="meta")
    c = torch.ops.helion_amd.moe_matmul_ogs(A, W, i32(3), i32(4), i32(10), 5)
    assert c.shape == (10, 12) and c.dtype == torch.bfloat16
    mx = torch.empty(32, 64, dtype=torch.float16, device="meta"); my = torch.empty(64, 48, dtype=torch.float16, device="meta")
    mo = torch.ops.helion_amd.matmul(mx, my, None, True, torch.float32, 0)
    assert mo.shape == (32, 48) and mo.dtype == torch.float32
    aq = torch.empty(2, 3, 100, 64, dtype=torch.bfloat16, device="meta"); ak = torch.empty(2, 3, 70, 64, dtype=torch.bfloat16, device="meta")
    ao = torch.ops.helion_amd.attention(aq, ak, ak)
    assert ao.shape == (2, 3, 100, 64) and ao.dtype == torch.bfloat16


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from helion_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "_LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_product_package_never_touches_the_oracle():
    """The oracle is the checker: nothing under helion_amd/ may import, read or run it (and importing the package must not
    pull it in as a side effect either)."""
    import pathlib
    import subprocess
    import sys

    root = pathlib.Path(__file__).resolve().parent.parent
    for f in (root / "helion_amd").rglob("*"):
        if f.suffix in (".py", ".hip", ".h", ".cpp"):
            assert "oracle" not in f.read_text(), f
    code = "import sys, helion_amd; assert not any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules), 'oracle imported'"
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-500:]


def test_product_package_never_touches_the_host_execution_model():
    """tests/sim (the kernel sources compiled for the CPU) is a checker like the oracle: nothing under helion_amd/ or in
    bench.py may refer to it, and the library the package loads is the hipcc-built one only."""
    import pathlib

    root = pathlib.Path(__file__).resolve().parent.parent
    for f in list((root / "helion_amd").rglob("*")) + [root / "bench.py"]:
        if f.suffix in (".py", ".hip", ".h", ".cpp"):
            text = f.read_text()
            assert "hx_sim" not in text and "hxsim" not in text and "tests.sim" not in text and "tests/sim" not in text, f
    from helion_amd import _lib
    assert _lib.lib_path().name == "libhx_kernels.so" and _lib.lib_path().parent.name == "helion_amd"


def test_the_inline_mfma_distance_scanner_sees_both_kinds_of_pair():
    """helion_amd/csrc/scan_mfma_hazards.py on a hand-made listing: an accumulator read 2 instructions after the MFMA that
    wrote it, and an MFMA 1 instruction after a vector-ALU write to one of its sources."""
    import importlib.util
    import pathlib
    path = pathlib.Path(__file__).resolve().parent.parent / "helion_amd" / "csrc" / "scan_mfma_hazards.py"
    spec = importlib.util.spec_from_file_location("scan_mfma_hazards", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    asm = """
_Z6kernelv:
	v_mfma_f32_16x16x32_bf16 a[4:7], v[10:13], v[20:23], a[4:7]
	s_nop 1
	v_accvgpr_read_b32 v1, a5
	ds_read_b128 v[30:33], v2
	v_mov_b32_e32 v31, v9
	v_mfma_f32_16x16x32_bf16 a[8:11], v[30:33], v[20:23], 0
	v_accvgpr_read_b32 v3, a100
.Lfunc_end0:
"""
    (name, n, d_read, d_src), = mod.scan(asm, "kernel", 16)
    assert (n, d_read, d_src) == (7, 2, 1)
    clean = asm.replace("a5", "a200").replace("v_mov_b32_e32 v31, v9", "s_nop 0")
    (_, _, d_read, d_src), = mod.scan(clean, "kernel", 16)
    assert d_read == 17 and d_src == 17   # nothing within the window
