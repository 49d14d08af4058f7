"""ctypes binding of the C-ABI library (include/lowp.h).

The library is built in-tree by g-core-gh_amd/build.py.  There is no CPU or
PyTorch fallback: if the library or a GPU is missing, calls raise.
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (must be imported first: it loads the HIP runtime the library binds to)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("LOWP_LIB") or os.path.join(_HERE, "_lib", "liblowp.so")

# enum lp_dtype
F32, BF16, E8M0, E4M3 = 0, 1, 2, 3
# enum lp_scale_mode
SCALE_POW2, SCALE_DIV, SCALE_MUL, SCALE_RCP, SCALE_RCP_POW2, SCALE_MUL_FLOOR = 0, 1, 2, 3, 4, 5
# enum lp_zero_rule
ZERO_NONE, ZERO_AMAX_TO_ONE, ZERO_SCALE_TO_ONE = 0, 1, 2
# enum lp_fp4_zero
FP4_POS_ZERO, FP4_NEG_ZERO = 0, 1
PAD_MIXED = 0              # lp_quant_fp8_colwise_t: 128-row padding up to 256 rows, 512 beyond

_i64, _p, _i32, _f32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float

# name -> (restype, argtypes); mirrors include/lowp.h one to one
PROTOTYPES = {
    "lp_version": (_i32, []),
    "lp_last_error": (ctypes.c_char_p, []),
    "lp_quant_fp8_block": (_i32, [_p, _i32, _i64, _i64, _i32, _i32, _i32, _f32, _i32, _p, _p, _i32, _p, _p]),
    "lp_quant_fp4_block": (_i32, [_p, _i32, _i64, _i64, _i32, _i32, _p, _p, _p, _p]),
    "lp_qdq_fp8_tile128": (_i32, [_p, _i64, _i64, _p, _p]),
    "lp_fp4_qat_to_fp8": (_i32, [_p, _i64, _i64, _p, _p, _p]),
    "lp_fp4_qdq_row32": (_i32, [_p, _i64, _p, _p, _p]),
    "lp_act_qdq_group": (_i32, [_p, _i64, _i32, _i32, _i32, _p, _p, _p]),
    "lp_dequant_fp8_block": (_i32, [_p, _p, _i32, _i64, _i64, _i32, _i32, _p, _i32, _p]),
    "lp_dequant_fp4_block": (_i32, [_p, _p, _i32, _i64, _i64, _i32, _i32, _i32, _p, _i32, _p]),
    "lp_fp4_to_fp8_rebase": (_i32, [_p, _p, _i64, _i64, _p, _p, _i32, _p]),
    "lp_fp4_to_fp8_amax": (_i32, [_p, _p, _i64, _i64, _i32, _f32, _i32, _p, _p, _i32, _p, _p]),
    "lp_gemm_fp8_block": (_i32, [_p, _p, _p, _p, _i32, _i64, _i64, _i64, _p, _i32, _p, _i64, _p]),
    "lp_gemm_fp8_block_static": (_i32, [_p, _p, _p, _p, _i32, _i64, _i64, _i64, _p, _i32, _p]),
    "lp_gemm_static_scratch_bytes": (_i64, []),
    "lp_gemm_nt": (_i32, [_p, _p, _i32, _i64, _i64, _i64, _p, _i32, _p]),
    "lp_gemm_fp8_rowscale": (_i32, [_p, _p, _p, _p, _i32, _i64, _i64, _i64, _p, _i32, _p]),
    "lp_gemm_fp8_rowscale_grouped": (_i32, [_p, _p, _p, _p, _i32, _p, _i32, _i32, _i32, _i64, _i64, _p, _i32, _p]),
    "lp_quant_fp8_colwise_t": (_i32, [_p, _i32, _i64, _i64, _p, _i32, _i64, _i32, _p, _p, _i32, _p]),
    "lp_gemm_fp8_grouped": (_i32, [_p, _p, _p, _p, _i32, _p, _i32, _i64, _i64, _i64, _p, _i32, _p]),
    "lp_gemm_fp8_grouped_nn": (_i32, [_p, _p, _p, _p, _i32, _p, _i32, _i64, _i64, _i64, _p, _i32, _p]),
    "lp_gemm_workspace_bytes": (_i64, [_i64, _i64, _i64]),
}

_lib = None


class LowpError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LowpError(
                f"{LIB_PATH} is missing: build it with `python g-core-gh_amd/build.py` "
                "(there is no CPU fallback for this path)")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error() -> str:
    return lib().lp_last_error().decode()


def check(rc: int, exc=LowpError):
    if rc != 0:
        raise exc(last_error() or f"lowp call failed with status {rc}")


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise LowpError("no GPU visible: the low-precision path runs on an MI355X only (no CPU fallback)")
    return torch.device("cuda", torch.cuda.current_device())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr() -> int:
    """The current stream of the current device as the handle the C ABI takes.  Through torch's raw accessor where it
    exists: building a Stream object per call cost 4 us of the 15 an eager decode GEMM call takes."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def to_device(t: torch.Tensor):
    """Return (tensor on the GPU, original device).  CPU inputs are staged through
    the GPU and results are moved back by the caller, so outputs follow inputs."""
    if t.is_cuda:
        return t, t.device
    dev = require_gpu()
    return t.to(dev), t.device


_SCALE_DTYPES = {torch.float32: F32, torch.bfloat16: BF16, torch.float8_e8m0fnu: E8M0}


def scale_code(dtype: torch.dtype) -> int:
    try:
        return _SCALE_DTYPES[dtype]
    except KeyError:
        raise TypeError(f"unsupported scale dtype {dtype}") from None
