"""Python side of the host execution model (tests/sim/hx_sim.h): loads tests/sim/libhx_sim.so - the kernel sources
compiled for the CPU behind the library's own C ABI - and hands out operand buffers that sit between inaccessible pages.
Used by the `not gpu` tests only; the package under helion_amd/ never touches it."""
from __future__ import annotations

import ctypes
import pathlib
import sys

import torch

SIM = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(SIM))
import build as _build  # noqa: E402

from helion_amd import _lib as _real  # noqa: E402  (for the signature table and the dtype tags only)

_c = ctypes
_lib = None


def load():
    global _lib
    if _lib is None:
        if not _build.is_current():
            _build.build(only_if_stale=True)
        lib = ctypes.CDLL(str(_build.LIB))
        for name, (res, args) in _real._SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        lib.hx_sim_alloc.restype, lib.hx_sim_alloc.argtypes = _c.c_void_p, [_c.c_size_t, _c.c_int]
        lib.hx_sim_free_all.restype, lib.hx_sim_free_all.argtypes = None, []
        lib.hx_sim_config.restype, lib.hx_sim_config.argtypes = None, [_c.c_int, _c.c_int, _c.c_int]
        lib.hx_sim_last_fault.restype, lib.hx_sim_last_fault.argtypes = _c.c_char_p, []
        lib.hx_sim_reset.restype, lib.hx_sim_reset.argtypes = None, []
        lib.hx_sim_counters.restype, lib.hx_sim_counters.argtypes = None, [_c.POINTER(_c.c_uint64)]
        lib.hx_sim_cvt_pk_fp8.restype, lib.hx_sim_cvt_pk_fp8.argtypes = _c.c_int, [_c.c_float, _c.c_float]
        lib.hx_sim_set_wg_reverse.restype, lib.hx_sim_set_wg_reverse.argtypes = _c.c_int, [_c.c_int]
        lib.hx_sim_work.restype, lib.hx_sim_work.argtypes = None, [_c.POINTER(_c.c_uint64), _c.c_int]
        lib.hx_sim_in_flight_source.restype, lib.hx_sim_in_flight_source.argtypes = None, [_c.c_void_p, _c.c_size_t]
        lib.hx_sim_set_check_lds.restype, lib.hx_sim_set_check_lds.argtypes = _c.c_int, [_c.c_int]
        lib.hx_sim_set_cus.restype, lib.hx_sim_set_cus.argtypes = _c.c_int, [_c.c_int]
        lib.hx_sim_selftest.restype, lib.hx_sim_selftest.argtypes = _c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int]
        _lib = lib
    return _lib


# the scheduling / DMA-landing variants a kernel must give the same answer under:
# (dma_lazy, wave_order, interleave)
VARIANTS = {"eager": (0, 0, 0), "lazy": (1, 0, 0), "lazy-reverse": (1, 1, 0), "eager-interleaved": (0, 1, 1), "lazy-interleaved": (1, 0, 1)}


class Arena:
    """Operand buffers for one test case.  `end_flush` puts the last byte of every buffer right before an inaccessible
    page (overruns fault at the first byte); otherwise the first byte sits right behind one (underruns do)."""

    def __init__(self, end_flush: bool = True):
        self.lib = load()
        self.end_flush = end_flush
        self._keep = []

    def empty(self, nbytes: int) -> torch.Tensor:
        nbytes = max(int(nbytes), 1)
        p = self.lib.hx_sim_alloc(nbytes, 1 if self.end_flush else 0)
        assert p, "hx_sim_alloc failed"
        raw = (_c.c_uint8 * nbytes).from_address(p)
        self._keep.append(raw)
        return torch.frombuffer(raw, dtype=torch.uint8)

    def put(self, t: torch.Tensor) -> torch.Tensor:
        """A copy of the contiguous tensor `t` in a guarded buffer, same dtype and shape."""
        t = t.contiguous()
        b = self.empty(t.numel() * t.element_size())
        b[: t.numel() * t.element_size()].copy_(t.view(torch.uint8).reshape(-1))
        return b[: t.numel() * t.element_size()].view(t.dtype).reshape(t.shape)

    def out(self, shape, dtype, fill=None) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        es = torch.empty((), dtype=dtype).element_size()
        b = self.empty(n * es)
        t = b[: n * es].view(dtype).reshape(shape)
        if fill is not None:
            t.view(torch.uint8).fill_(fill)
        return t

    def close(self):
        self._keep.clear()
        self.lib.hx_sim_free_all()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    lib = load()
    msg = lib.hx_last_error().decode("utf-8", "replace")
    fault = lib.hx_sim_last_fault().decode("utf-8", "replace")
    lib.hx_sim_reset()
    raise AssertionError(f"{what}: rc {rc}: {msg} | {fault}")


def configure(variant: str) -> None:
    load().hx_sim_config(*VARIANTS[variant])


class features:
    """with simlib.features(mask): the opt-in kernel paths of the mask are on inside the block."""

    def __init__(self, mask: int):
        self.mask = mask

    def __enter__(self):
        self.old = load().hx_set_features(self.mask)

    def __exit__(self, *exc):
        load().hx_set_features(self.old)


class cus:
    """with simlib.cus(n): the modelled chip has n compute units (1 .. 63, or 256) inside the block."""

    def __init__(self, n: int):
        self.n = n

    def __enter__(self):
        self.old = load().hx_sim_set_cus(self.n)

    def __exit__(self, *exc):
        load().hx_sim_set_cus(self.old)


class workgroups_last_to_first:
    """with simlib.workgroups_last_to_first(): the workgroups of a launch run in reverse order, each to completion, so
    workgroup 0 is the last to start (a workgroup that waits for something workgroup 0 does can only give up)."""

    def __enter__(self):
        self.old = load().hx_sim_set_wg_reverse(1)

    def __exit__(self, *exc):
        load().hx_sim_set_wg_reverse(self.old)


def work(reset: bool = True) -> dict:
    """What the launches since the last reset did: wave-level MFMA instructions, bytes moved global -> LDS by DMA, LDS
    bytes read / written by the kernels' own loads and stores (transposing reads included), workgroup barriers, workgroups;
    the most DMA bytes one workgroup had issued and not yet waited for, and the mean of that figure right after its waits
    (the window of bytes the code lets be in flight: its upper and lower edge)."""
    c = (_c.c_uint64 * 9)()
    load().hx_sim_work(c, int(reset))
    d = dict(zip(("mfma", "dma_bytes", "lds_read", "lds_write", "barriers", "workgroups", "dma_in_flight_max"), (int(x) for x in c)))
    d["dma_in_flight_after_waits"] = c[7] / c[8] if c[8] else 0.0
    return d
