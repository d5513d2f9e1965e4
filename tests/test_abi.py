"""The C-ABI library loads, exports every symbol include/hx_kernels.h declares, and rejects bad
arguments before touching the GPU (so these run without one)."""
import ctypes
import pathlib
import re

import pytest

from helion_amd import _lib

ROOT = pathlib.Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "hx_kernels.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hx_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(_lib.exported_symbols())


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_lib.lib_path()))
    for name in _declared_symbols():
        assert hasattr(lib, name), f"{name} declared in include/hx_kernels.h but not exported"
    assert _lib.load().hx_version() >= 1


def test_gemm_argument_errors_are_reported_without_a_launch():
    lib = _lib.load()
    assert lib.hx_fp8_gemm(None, None, None, -1, 4, 4, 4, 1, 4, 4, None, None, 0, None, 0, None) == -1
    assert b"negative" in lib.hx_last_error()
    assert lib.hx_fp8_gemm(None, None, None, 4, 4, 4, 4, 1, 4, 4, None, None, 0, None, 0, None) == -1
    assert b"null" in lib.hx_last_error()
    assert lib.hx_fp8_gemm(1, 1, 1, 4, 4, 4, 4, 1, 4, 4, None, None, 9, None, 0, None) == -1  # bad dtype tag
    assert lib.hx_fp8_gemm(1, 1, 1, 4, 4, 8, 4, 1, 8, 4, None, None, 0, None, 0, None) == -1  # lda < K
    assert lib.hx_fp8_gemm(None, None, None, 0, 4, 4, 4, 1, 4, 4, None, None, 0, None, 0, None) == 0  # empty
    with pytest.raises(ValueError):
        _lib.check(-1, "x")


def test_gemm_path_selection():
    lib = _lib.load()
    A = 1 << 20  # any 16-byte aligned fake address; the query never dereferences
    assert lib.hx_fp8_gemm_path(8192, 8192, 8192, 8192, 1, 8192, 8192, A, A, A) == 1
    assert lib.hx_fp8_gemm_path(16, 28672, 8192, 8192, 1, 8192, 28672, A, A, A) == 2
    assert lib.hx_fp8_gemm_path(1, 512, 256, 256, 1, 256, 512, A, A, A) == 2
    assert lib.hx_fp8_gemm_path(32, 28672, 8192, 8192, 1, 8192, 28672, A, A, A) == 2   # up to 32 rows when K <= 8192
    assert lib.hx_fp8_gemm_path(33, 28672, 8192, 8192, 1, 8192, 28672, A, A, A) == 5   # a decode batch: 128-column tiles
    assert lib.hx_fp8_gemm_path(2048, 2048, 2048, 2048, 1, 2048, 2048, A, A, A) == 5   # 64 tiles of 256x256 would idle the chip
    assert lib.hx_fp8_gemm_path(4096, 4096, 4096, 4096, 1, 4096, 4096, A, A, A) == 1
    # tile choice by estimated rounds: two rounds of 128x128 tiles beat one half-empty round of 256x256 tiles when K is
    # long, but not five rounds against two when K is two k-tiles
    assert lib.hx_fp8_gemm_path(1024, 7168, 8192, 8192, 1, 8192, 7168, A, A, A) == 5
    assert lib.hx_fp8_gemm_path(2048, 4096, 4096, 4096, 1, 4096, 4096, A, A, A) == 5
    assert lib.hx_fp8_gemm_path(8192, 1280, 8192, 8192, 1, 8192, 1280, A, A, A) == 1
    assert lib.hx_fp8_gemm_path(4096, 8192, 7168, 7168, 1, 7168, 8192, A, A, A) == 1
    assert lib.hx_fp8_gemm_path(4000, 4100, 256, 256, 1, 256, 4100, A, A, A) == 3
    assert lib.hx_fp8_gemm_path(256, 256, 256, 256, 256, 1, 256, A, A, A) == 4  # row-major B, read in place
    assert lib.hx_fp8_gemm_path(16, 256, 256, 256, 256, 1, 256, A, A, A) == 0   # row-major B for the skinny shape: via workspace
    assert lib.hx_fp8_gemm_path(100, 72, 128, 128, 72, 1, 72, A, A, A) == 0     # row-major B, N % 16 != 0
    assert lib.hx_fp8_gemm_path(100, 70, 50, 50, 1, 50, 70, A, A, A) == 0  # ragged K
    assert lib.hx_fp8_gemm_path(5000, 5000, 1024, 1024, 1, 1024, 5000, A, A, A) == 3  # ragged M/N: guarded edge tiles
    assert lib.hx_fp8_gemm_path(1000, 1000, 1040, 1040, 1, 1040, 1000, A, A, A) == 3  # K % 128 != 0
    assert lib.hx_fp8_gemm_workspace_bytes(256, 512, 384, 512, 1) == 0          # row-major B the tile kernel reads in place
    assert lib.hx_fp8_gemm_workspace_bytes(8, 512, 384, 512, 1) == 512 * 384    # skinny shape: transpose scratch
    assert lib.hx_fp8_gemm_workspace_bytes(256, 512, 384, 1, 384) == 0
    # column-major B: split-K partial sums only for few 128-column tiles and a long K, never for the skinny shapes
    assert lib.hx_fp8_gemm_workspace_bytes(1024, 1280, 8192, 1, 8192) == 3 * 1024 * 1280 * 4
    assert lib.hx_fp8_gemm_workspace_bytes(64, 2048, 8192, 1, 8192) == 8 * 64 * 2048 * 4
    assert lib.hx_fp8_gemm_workspace_bytes(1024, 1024, 1024, 1, 1024) == 0
    assert lib.hx_fp8_gemm_workspace_bytes(8192, 8192, 8192, 1, 8192) == 0
    assert lib.hx_fp8_gemm_workspace_bytes(16, 2048, 8192, 1, 8192) == 0
    assert lib.hx_fp8_gemm_workspace_bytes(64, 28672, 8192, 1, 8192) == 0
    assert lib.hx_fp8_gemm_workspace_bytes(300, 520, 2048 + 16, 1, 2064) == 0   # K % 128 != 0: the edge kernel, no split
    assert lib.hx_fp8_gemm_path(256, 256, 256, 256, 1, 256, 256, A + 1, A, A) == 0  # misaligned


def test_attention_and_moe_argument_errors():
    lib = _lib.load()
    assert lib.hx_fp8_attention(1, 1, 1, 1, -1, 64, 64, 0, 64, 1, 3, 1, None) == -1
    assert lib.hx_fp8_attention(16, 16, 16, 16, 2, 128, 320, 0, 128, 1, 3, 1, None) == -2  # head dim > 256: no kernel takes it
    assert b"unsupported shape" in lib.hx_last_error()
    assert lib.hx_fp8_attention(16, 16, 16, 16, 2, 128, 64, 0, 128, 1, 1, 1, None) == -1  # bf16 output not offered
    assert lib.hx_fp8_attention(None, None, None, None, 0, 128, 64, 0, 128, 1, 3, 1, None) == 0
    assert lib.hx_moe_workspace_bytes(1000, 30) >= 1000
    assert lib.hx_moe_grouped_gemm(16, 16, 16, 16, 16, 16, 8, 8, 8, 2, 8, 2, None, 0, None) == -1  # f32 tag
    assert lib.hx_moe_grouped_gemm(16, 16, 16, 16, 16, 16, 8, 8, 8, 2, 8, 1, None, 0, None) == -3  # no workspace
    assert b"workspace" in lib.hx_last_error()
    assert lib.hx_moe_routing(16, 1, 100, 513, 16, 16, 16, 16, None, 0, None) == -2  # more experts than the kernel's table holds
    assert lib.hx_moe_routing(None, 1, 100, 8, 16, 16, 16, 16, None, 0, None) == -1
    assert lib.hx_moe_routing(16, 1, -1, 8, 16, 16, 16, 16, None, 0, None) == -1
    assert lib.hx_moe_routing_workspace_bytes(32768, 8) == 0 and lib.hx_moe_routing_workspace_bytes(1 << 20, 8) == 64 * 8 * 4
    assert lib.hx_moe_topk_workspace_bytes(1000, 2, 30) >= lib.hx_moe_workspace_bytes(2000, 30) + 2000 * 4
    assert lib.hx_moe_topk_matmul(16, 16, 16, 16, 1, 8, 0, 8, 8, 2, 1, None, 0, None) == -1  # top_k < 1
    assert lib.hx_moe_topk_matmul(16, 16, 16, 16, 1, 8, 2, 8, 8, 2, 1, None, 0, None) == -3  # no workspace


def test_cast_and_quantize_argument_errors():
    lib = _lib.load()
    assert lib.hx_cast_e4m3(16, 16, -1, 0, None, None) == -1
    assert lib.hx_cast_e4m3(16, 16, 8, 3, None, None) == -1      # e4m3 is not a source type
    assert lib.hx_cast_e4m3(None, 16, 8, 0, None, None) == -1
    assert lib.hx_cast_e4m3(24, 16, 8, 0, None, None) == -2      # misaligned
    assert lib.hx_cast_e4m3(None, None, 0, 0, None, None) == 0
    assert lib.hx_fp8_attention_preprocess(16, 16, None, 16, 16, 16, 8, 1, None) == -1
    assert lib.hx_fp8_quantize_workspace_bytes(1 << 20) >= 16 + 4
    assert lib.hx_fp8_quantize(16, 16, 8, 0, None, 16, 1 << 20, None) == -1   # no scale_out
    assert lib.hx_fp8_quantize(16, 16, 8, 0, 16, None, 0, None) == -3


def test_sibling_argument_errors_are_reported_without_a_launch():
    lib = _lib.load()
    A = 1 << 20
    assert lib.hx_matmul(None, None, None, -1, 4, 4, 4, 4, 1, 4, None, 0, 0, 1, 1, 1, None, 0, None) == -1
    assert lib.hx_matmul(A, A, A, 4, 4, 4, 4, 4, 1, 4, None, 0, 0, 3, 3, 1, None, 0, None) == -1        # e4m3 operands: not this entry
    assert lib.hx_matmul(A, A, A, 4, 4, 4, 4, 4, 1, 4, None, 0, 0, 1, 0, 1, None, 0, None) == -1        # bf16 in, fp16 out
    assert lib.hx_matmul(A, A, A, 4, 4, 8, 4, 4, 1, 4, None, 0, 0, 1, 1, 1, None, 0, None) == -1        # lda < K
    assert lib.hx_matmul(A, A, A, 256, 256, 4096, 4096, 256, 1, 256, None, 0, 0, 1, 1, 8, None, 0, None) == -3   # forced split, no workspace
    assert lib.hx_matmul(None, None, None, 0, 4, 4, 4, 4, 1, 4, None, 0, 0, 1, 1, 1, None, 0, None) == 0
    assert lib.hx_matmul_path(256, 256, 256, 256, 256, 1, 256, 1, A, A, A, None) == 1
    assert lib.hx_matmul_path(256, 256, 256, 256, 1, 256, 256, 1, A, A, A, None) == 1                    # column-major y
    assert lib.hx_matmul_path(256, 256, 250, 256, 256, 1, 256, 1, A, A, A, None) == 0                    # K % 64
    assert lib.hx_matmul_path(256, 256, 256, 256, 256, 1, 256, 2, A, A, A, None) == 0                    # fp32 operands
    assert lib.hx_matmul_splits(64, 64, 32768, 32768, 64, 1, 64, 0, 0) > 1
    assert lib.hx_matmul_splits(8192, 8192, 8192, 8192, 8192, 1, 8192, 1, 0) == 1
    assert lib.hx_matmul_workspace_bytes(64, 64, 32768, 32768, 64, 1, 64, 0, 0, 0, 4) == 4 * 64 * 64 * 4
    assert lib.hx_matmul_workspace_bytes(8192, 8192, 8192, 8192, 8192, 1, 8192, 1, 1, 1, 1) == 0
    assert lib.hx_attention(None, None, None, None, -1, 4, 4, 64, 0, 1, None) == -1
    assert lib.hx_attention(A, A, A, A, 2, 64, 0, 64, 0, 1, None) == -1                                     # no keys
    assert lib.hx_attention(A, A, A, A, 2, 64, 64, 64, 0, 3, None) == -1                                    # e4m3: not this entry
    assert lib.hx_attention(A, A, A, A, 2, 64, 64, 320, 0, 2, None) == -2                                   # fp32 head dim > 256
    assert lib.hx_attention(None, None, None, None, 0, 64, 64, 64, 0, 1, None) == 0
    assert lib.hx_attention_path(2, 100, 70, 128, 1, A, A, A, A) == 1
    assert lib.hx_attention_path(2, 100, 70, 96, 1, A, A, A, A) == 0
    assert lib.hx_attention_path(2, 100, 70, 128, 2, A, A, A, A) == 0


def test_moe_path_selection():
    """Host logic only: which grouped-GEMM kernel a shape gets (the query never dereferences its pointers)."""
    lib = _lib.load()
    A = 1 << 20
    assert lib.hx_moe_path(32768, 4096, 14336, 8, 1, A, A, A) == 3     # C5: 256-row tiles
    assert lib.hx_moe_path(4000, 4096, 1024, 8, 1, A, A, A) == 2       # < 512 rows per expert: 128-row tiles
    assert lib.hx_moe_path(2000, 4096, 14336, 64, 1, A, A, A) == 2
    assert lib.hx_moe_path(16, 4096, 14336, 8, 1, A, A, A) == 1        # a decode step: 32 rows in all
    assert lib.hx_moe_path(1000, 504, 200, 30, 1, A, A, A) == 4        # K % 64 != 0, K % 8 == 0: zero-filled last k-tile
    assert lib.hx_moe_path(1000, 500, 200, 30, 1, A, A, A) == 5        # the reference's own check shape (examples/moe_matmul_ogs.py:186): K even
    assert lib.hx_moe_path(1000, 501, 200, 30, 1, A, A, A) == 0        # odd K: rows of A not even 4-byte aligned
    assert lib.hx_moe_path(1000, 512, 204, 30, 1, A, A, A) == 0        # N % 8 != 0
    assert lib.hx_moe_path(1000, 512, 200, 30, 1, A + 2, A, A) == 0    # misaligned A
    assert lib.hx_moe_path(100, 64, 64, 4, 2, A, A, A) in (1, 2)       # top-k through a_div: still an MFMA kernel


def test_fp8_attention_path_selection():
    lib = _lib.load()
    A = 1 << 20
    assert lib.hx_fp8_attention_path(128, 4096, 128, 4096, 1, A, A, A, A) == 1   # C4, v as [D][S]
    assert lib.hx_fp8_attention_path(128, 4096, 128, 1, 128, A, A, A, A) == 1    # v as the reference's preprocessing leaves it
    assert lib.hx_fp8_attention_path(2, 208, 128, 208, 1, A, A, A, A) == 1       # partial last key tile
    assert lib.hx_fp8_attention_path(2, 200, 128, 1, 128, A, A, A, A) == 1
    assert lib.hx_fp8_attention_path(2, 200, 128, 200, 1, A, A, A, A) == 0       # [D][S] rows come in 16-byte pieces: S % 16
    assert lib.hx_fp8_attention_path(2, 128, 64, 128, 1, A, A, A, A) == 1
    assert lib.hx_fp8_attention_path(2, 128, 96, 128, 1, A, A, A, A) == 0        # (the Python op zero-pads such heads to 128)
    assert lib.hx_fp8_attention_path(2, 128, 256, 128, 1, A, A, A, A) == 0
    assert lib.hx_fp8_attention_path(2, 128, 128, 128, 1, A + 8, A, A, A) == 0   # misaligned q


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 with nothing but the standard headers, and a C program
    that calls a query function must link against the built library and run without a GPU."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    root = pathlib.Path(__file__).resolve().parent.parent
    src = tmp_path / "abi.c"
    src.write_text('#include <stdio.h>\n#include "hx_kernels.h"\n'
                   "int main(void) {\n"
                   "  if (hx_version() <= 0) return 1;\n"
                   "  if (hx_fp8_gemm_workspace_bytes(8192, 8192, 8192, 1, 8192) != 0) return 2;\n"
                   "  if (hx_fp8_gemm(0, 0, 0, -1, 1, 1, 1, 1, 1, 1, 0, 0, 1, 0, 0, 0) >= 0) return 3;  /* negative size: an error, no launch */\n"
                   '  printf("%s\\n", hx_last_error());\n'
                   "  return 0;\n}\n")
    lib = _lib.lib_path()
    exe = tmp_path / "abi"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", str(root / "include"), str(src), "-o", str(exe),
                    str(lib), f"-Wl,-rpath,{lib.parent}"], check=True, capture_output=True, text=True, timeout=120)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stderr[-300:])
    assert "hx_fp8_gemm" in r.stdout
