"""ctypes binding of the measurement / self-test library (include/lowp_probe.h, _lib/liblowp_probe.so).

Used by the tests and the benchmark only: no wrapper of the product path imports this module.
"""
from __future__ import annotations

import ctypes
import os

import torch

from . import _abi

LIB_PATH = os.environ.get("LOWP_PROBE_LIB") or os.path.join(os.path.dirname(_abi.LIB_PATH), "liblowp_probe.so")

_i64, _p, _i32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int

# name -> (restype, argtypes); mirrors include/lowp_probe.h one to one
PROTOTYPES = {
    "lp_probe_last_error": (ctypes.c_char_p, []),
    "lp_selftest": (_i32, [_i32, _p, _p]),
    "lp_probe_stream": (_i32, [_p, _i64, _p, _i64, _i32, _p]),
    "lp_probe_mfma": (_i32, [_i32, _i32, _p, _i32, _p]),
    "lp_probe_copy": (_i32, [_i32, _i32, _i32, _p, _i64, _i64, _p, _i32, _p]),
    "lp_debug_cast": (_i32, [_i32, _p, _p, _i64, _p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise _abi.LowpError(f"{LIB_PATH} is missing: build it with `python g-core-gh_amd/build.py`")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc: int):
    if rc != 0:
        raise _abi.LowpError(lib().lp_probe_last_error().decode() or f"probe call failed with status {rc}")


def selftest(which: int) -> int:
    """Number of inputs on which a gfx950 conversion instruction differs from the library's software cast."""
    dev = _abi.require_gpu()
    out = torch.zeros(1, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        check(lib().lp_selftest(which, out.data_ptr(), _abi.stream_ptr()))
    return int(out.item())


def debug_cast(kind: int, x: torch.Tensor) -> torch.Tensor:
    dev = _abi.require_gpu()
    xg = x.to(dev, torch.float32).contiguous()
    out = torch.empty(xg.shape, dtype=torch.int16 if kind == 3 else torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(lib().lp_debug_cast(kind, xg.data_ptr(), out.data_ptr(), xg.numel(), _abi.stream_ptr()))
    return out.cpu()
