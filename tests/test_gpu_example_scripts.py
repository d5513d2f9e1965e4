"""The example scripts' own entry points (`check` / `main` of examples/fp8_gemm.py:95-119, examples/fp8_attention.py:260-295,
examples/moe_matmul_ogs.py:152-186, examples/matmul.py:75-148, examples/matmul_split_k.py:72-124,
examples/attention.py:104-156) run against the package: kernel vs the script's torch baseline at the script's
tolerances, which is what the reference's test_examples does through run_example."""
import importlib

import pytest
import torch

# the package re-exports functions under the modules' names, so take the modules themselves
fp8_gemm, fp8_attention, moe_matmul_ogs, matmul, matmul_split_k, attention = (
    importlib.import_module(f"helion_amd.{m}")
    for m in ("fp8_gemm", "fp8_attention", "moe_matmul_ogs", "matmul", "matmul_split_k", "attention"))

pytestmark = pytest.mark.gpu


def test_fp8_gemm_main():
    torch.manual_seed(0)
    fp8_gemm.main()


def test_fp8_attention_main():
    fp8_attention.main()


def test_moe_matmul_ogs_main():
    torch.manual_seed(0)
    moe_matmul_ogs.main()


def test_matmul_main():
    torch.manual_seed(0)
    matmul.main()


def test_matmul_split_k_main():
    torch.manual_seed(0)
    matmul_split_k.main()


def test_attention_main():
    torch.manual_seed(0)
    attention.main()
