"""ctypes binding of libhx_kernels.so (the C ABI declared in include/hx_kernels.h).

There is no fallback: if the shared object is missing, every entry point raises.  Build it with
``python -m helion_amd.build`` (hipcc, gfx950)."""
from __future__ import annotations

import ctypes
import pathlib

HX_F16, HX_BF16, HX_F32, HX_E4M3 = 0, 1, 2, 3
HX_FEATURE_SKINNY_ROWMAJOR = 1
HX_FEATURE_FP8_GEMM_ANY_K = 2
HX_FEATURE_ATTENTION_D256 = 4
HX_FEATURE_FP8_GEMM_PERSISTENT = 8
HX_FEATURE_FP8_GEMM_DECODE_RING = 16
HX_FEATURE_ROUTING_WIDE = 32
HX_FEATURE_MOE_PERSISTENT = 64
HX_FEATURE_MATMUL_PERSISTENT = 128
HX_FEATURE_MOE_ANY_SHAPE = 256

_LIB_PATH = pathlib.Path(__file__).resolve().parent / "libhx_kernels.so"
_lib = None

_c = ctypes
_SIGNATURES = {
    "hx_version": (_c.c_int, []),
    "hx_last_error": (_c.c_char_p, []),
    "hx_set_features": (_c.c_uint, [_c.c_uint]),
    "hx_get_features": (_c.c_uint, []),
    "hx_fp8_gemm": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
         _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_size_t, _c.c_void_p],
    ),
    "hx_fp8_gemm_workspace_bytes": (_c.c_size_t, [_c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64]),
    "hx_fp8_gemm_path": (
        _c.c_int,
        [_c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p,
         _c.c_void_p, _c.c_void_p],
    ),
    "hx_fp8_attention": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
         _c.c_int64, _c.c_int, _c.c_int, _c.c_void_p],
    ),
    "hx_fp8_attention_path": (_c.c_int, [_c.c_int64] * 5 + [_c.c_void_p] * 4),
    "hx_moe_path": (_c.c_int, [_c.c_int64] * 5 + [_c.c_void_p] * 3),
    "hx_moe_grouped_gemm": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64,
         _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_void_p, _c.c_size_t, _c.c_void_p],
    ),
    "hx_moe_workspace_bytes": (_c.c_size_t, [_c.c_int64, _c.c_int64]),
    "hx_moe_workspace_bytes_shape": (_c.c_size_t, [_c.c_int64] * 4),
    "hx_moe_grouped_gemm_static": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64,
         _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_void_p],
    ),
    "hx_moe_routing": (
        _c.c_int,
        [_c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
         _c.c_size_t, _c.c_void_p],
    ),
    "hx_moe_routing_workspace_bytes": (_c.c_size_t, [_c.c_int64, _c.c_int64]),
    "hx_moe_topk_matmul": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
         _c.c_int64, _c.c_int, _c.c_void_p, _c.c_size_t, _c.c_void_p],
    ),
    "hx_moe_topk_workspace_bytes": (_c.c_size_t, [_c.c_int64, _c.c_int64, _c.c_int64]),
    "hx_cast_e4m3": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_void_p, _c.c_void_p]),
    "hx_fp8_attention_preprocess": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_void_p],
    ),
    "hx_fp8_quantize": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_size_t, _c.c_void_p],
    ),
    "hx_fp8_quantize_workspace_bytes": (_c.c_size_t, [_c.c_int64]),
    "hx_matmul": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p] + [_c.c_int64] * 7 + [_c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.c_int,
                                                                      _c.c_void_p, _c.c_size_t, _c.c_void_p],
    ),
    "hx_matmul_workspace_bytes": (_c.c_size_t, [_c.c_int64] * 7 + [_c.c_int, _c.c_int, _c.c_int, _c.c_int]),
    "hx_matmul_splits": (_c.c_int, [_c.c_int64] * 7 + [_c.c_int, _c.c_int]),
    "hx_attention": (_c.c_int, [_c.c_void_p] * 4 + [_c.c_int64] * 5 + [_c.c_int, _c.c_void_p]),
    "hx_attention_path": (_c.c_int, [_c.c_int64] * 4 + [_c.c_int] + [_c.c_void_p] * 4),
    "hx_clock_probe": (_c.c_int, [_c.c_void_p, _c.c_int64, _c.c_void_p]),
    "hx_matmul_path": (_c.c_int, [_c.c_int64] * 7 + [_c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p]),
}


def lib_path() -> pathlib.Path:
    return _LIB_PATH


def exported_symbols() -> list[str]:
    return list(_SIGNATURES)


def load():
    """Load (once) and return the ctypes handle; raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(
                f"{_LIB_PATH} is missing: the HIP kernels are not built. Run `python -m helion_amd.build` "
                "(needs hipcc; cross-compiles for gfx950 without a GPU). There is no CPU or PyTorch fallback."
            )
        lib = ctypes.CDLL(str(_LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a non-zero C-ABI return into a Python exception (ValueError for argument errors)."""
    if rc == 0:
        return
    msg = load().hx_last_error().decode("utf-8", "replace")
    if rc < 0:
        raise ValueError(f"{what}: {msg} (code {rc})")
    raise RuntimeError(f"{what}: {msg} (hipError {rc})")


def set_features(mask: int) -> int:
    """Switch opt-in kernel paths on (HX_FEATURE_* bits, see include/hx_kernels.h); returns the previous mask.  These are
    paths that have passed the CPU-side checks but not yet a run on the hardware, which is why they default to off."""
    return load().hx_set_features(int(mask))
