"""MI355X (gfx950) kernels behind the Helion example entry points fp8_gemm, fp8_attention_kernel and moe_matmul_ogs,
and their 16-bit siblings matmul, matmul_split_k and attention.  Importing the package does not load the HIP library; the first op call does, and
fails loudly if it has not been built."""
from ._lib import HX_FEATURE_ATTENTION_D256, HX_FEATURE_FP8_GEMM_DECODE_RING, HX_FEATURE_FP8_GEMM_PERSISTENT, HX_FEATURE_MATMUL_PERSISTENT, HX_FEATURE_MOE_ANY_SHAPE, HX_FEATURE_MOE_PERSISTENT, HX_FEATURE_ROUTING_WIDE, HX_FEATURE_FP8_GEMM_ANY_K, HX_FEATURE_SKINNY_ROWMAJOR, set_features
from .attention import attention, attention_dynamic
from .fp8_attention import (fp8_attention_kernel, fp8_attention_pytorch, fp8_attention_tritonbench,
                            preprocess_fp8_attention_inputs)
from .fp8_gemm import (fp8_gemm, fp8_gemm_scaled, fp8_gemm_tritonbench, fp8_quantize_per_tensor,
                       reference_fp8_gemm_pytorch)
from .matmul import matmul, matmul_tritonbench
from .matmul_split_k import matmul_split_k, matmul_split_k_tritonbench
from .moe_matmul_ogs import (moe_matmul_ogs, moe_matmul_ogs_helion_kernel_args_gen, moe_matmul_ogs_reference,
                             moe_matmul_topk, moe_routing)

__all__ = [
    "fp8_gemm", "fp8_gemm_scaled", "fp8_gemm_tritonbench", "fp8_quantize_per_tensor", "reference_fp8_gemm_pytorch",
    "fp8_attention_kernel", "fp8_attention_pytorch", "fp8_attention_tritonbench", "preprocess_fp8_attention_inputs",
    "moe_matmul_ogs", "moe_matmul_ogs_helion_kernel_args_gen", "moe_matmul_ogs_reference",
    "moe_matmul_topk", "moe_routing",
    "set_features", "HX_FEATURE_SKINNY_ROWMAJOR", "HX_FEATURE_FP8_GEMM_ANY_K", "HX_FEATURE_ATTENTION_D256", "HX_FEATURE_FP8_GEMM_PERSISTENT", "HX_FEATURE_FP8_GEMM_DECODE_RING", "HX_FEATURE_ROUTING_WIDE", "HX_FEATURE_MOE_PERSISTENT", "HX_FEATURE_MATMUL_PERSISTENT", "HX_FEATURE_MOE_ANY_SHAPE",
    "attention", "attention_dynamic", "matmul", "matmul_tritonbench", "matmul_split_k", "matmul_split_k_tritonbench",
]
