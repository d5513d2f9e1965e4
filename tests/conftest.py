import ctypes
import os
import pathlib
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_runtest_logstart(nodeid, location):
    """Names every GPU test on the real stderr before it starts (unbuffered, past pytest's capture): if a kernel takes the
    process or the box down, the last line printed says which case it was."""
    if "test_gpu_" in nodeid or "test_zz_no_alloc" in nodeid or "wip_gpu_" in nodeid:
        try:
            os.write(2, f"[gpu-test] {nodeid}\n".encode())
        except OSError:
            pass


@pytest.fixture(scope="session")
def oracle_c():
    """ctypes handle of the C restatement (oracle/ref_c.c), built on demand with gcc."""
    from oracle import build as obuild

    lib = ctypes.CDLL(str(obuild.build(force=False)))
    c = ctypes
    lib.orc_e4m3_decode.restype = c.c_float
    lib.orc_e4m3_decode.argtypes = [c.c_uint8]
    lib.orc_e4m3_encode.restype = c.c_uint8
    lib.orc_e4m3_encode.argtypes = [c.c_float]
    lib.orc_fp8_gemm_f64.restype = None
    lib.orc_fp8_gemm_f64.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_int]
    lib.orc_fp8_attention_f64.restype = None
    lib.orc_fp8_attention_f64.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_void_p, c.c_int, c.c_int]
    lib.orc_moe_f64.restype = None
    lib.orc_moe_f64.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_void_p, c.c_int, c.c_int, c.c_int, c.c_int]
    return lib
