"""ctypes front end for the scalar C oracle (oracle/lowp_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests, the smoke check and the
cpu-baseline leg of the benchmark, never by the product package.  All entry
points take and return numpy arrays.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liblowp_oracle.so")

POW2, DIV, MUL = 0, 1, 2
SCALE_RCP, SCALE_RCP_POW2, SCALE_MUL_FLOOR = 3, 4, 5
ZERO_NONE, ZERO_AMAX_TO_ONE, ZERO_SCALE_TO_ONE = 0, 1, 2
LOG2_LIBM, LOG2_EXACT = 0, 1


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a second or two)."""
    src = os.path.join(_HERE, "lowp_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, p, i32, f32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        for name in ("orc_bulk_f32_to_e4m3fn", "orc_bulk_e4m3fn_to_f32", "orc_bulk_f32_to_bf16",
                     "orc_bulk_f32_to_e8m0", "orc_bulk_e8m0_to_f32"):
            getattr(L, name).argtypes = [p, p, i64]
            getattr(L, name).restype = None
        L.orc_pow2_exponent.argtypes = [f32, i32]
        L.orc_pow2_exponent.restype = i32
        L.orc_e2m1_value.argtypes = [i32, i32]
        L.orc_e2m1_value.restype = f32
        L.orc_quant_fp8_block.argtypes = [p, i64, i64, i32, i32, i32, f32, i32, i32, p, p, p]
        L.orc_quant_fp8_block.restype = i64
        L.orc_quant_fp4_block.argtypes = [p, i64, i64, i32, i32, i32, p, p]
        L.orc_quant_fp4_block.restype = i64
        L.orc_dequant_fp8_block.argtypes = [p, p, i64, i64, i32, i32, p, p]
        L.orc_dequant_fp8_block.restype = None
        L.orc_fp4_dequant.argtypes = [p, p, i64, i64, i32, i32, i32, p, p]
        L.orc_fp4_dequant.restype = None
        L.orc_fp4_to_e4m3_rebase.argtypes = [p, p, i64, i64, p, p, p]
        L.orc_fp4_to_e4m3_rebase.restype = None
        L.orc_gemm_fp8_block.argtypes = [p, p, p, p, i64, i64, i64, p]
        L.orc_gemm_fp8_block.restype = None
        _lib = L
    return _lib


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def _bulk(name, x, in_dt, out_dt):
    x = np.ascontiguousarray(x, dtype=in_dt)
    y = np.empty(x.shape, dtype=out_dt)
    getattr(lib(), name)(_ptr(x), _ptr(y), x.size)
    return y


def f32_to_e4m3fn(x):
    return _bulk("orc_bulk_f32_to_e4m3fn", x, np.float32, np.uint8)


def e4m3fn_to_f32(x):
    return _bulk("orc_bulk_e4m3fn_to_f32", x, np.uint8, np.float32)


def f32_to_bf16(x):
    return _bulk("orc_bulk_f32_to_bf16", x, np.float32, np.uint16)


def f32_to_e8m0(x):
    return _bulk("orc_bulk_f32_to_e8m0", x, np.float32, np.uint8)


def e8m0_to_f32(x):
    return _bulk("orc_bulk_e8m0_to_f32", x, np.uint8, np.float32)


def pow2_exponent(r: float, kind: int) -> int:
    return lib().orc_pow2_exponent(ctypes.c_float(r), kind)


def e2m1_value(code: int, neg_zero: int) -> float:
    return lib().orc_e2m1_value(code, neg_zero)


def quant_fp8_block(x, bm, bn, mode, amax_floor=0.0, zero_rule=ZERO_NONE, log2_kind=LOG2_LIBM):
    """x fp32 [rows, cols] -> (codes u8 [rows, cols], scale f32 [rows/bm, cols/bn],
    scale e8m0 bytes, number of NaN inputs)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    assert rows % bm == 0 and cols % bn == 0
    q = np.empty((rows, cols), np.uint8)
    s = np.empty((rows // bm, cols // bn), np.float32)
    sb = np.empty((rows // bm, cols // bn), np.uint8)
    nan = lib().orc_quant_fp8_block(_ptr(x), rows, cols, bm, bn, mode, ctypes.c_float(amax_floor),
                                    zero_rule, log2_kind, _ptr(q), _ptr(s), _ptr(sb))
    return q, s, sb, nan


def quant_fp4_block(x, bm=1, bn=32, log2_kind=LOG2_LIBM):
    """x fp32 [rows, cols] -> (packed u8 [rows, cols/2], scale e8m0 bytes [rows/bm, cols/bn], NaN count)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    assert rows % bm == 0 and cols % bn == 0 and cols % 2 == 0
    packed = np.empty((rows, cols // 2), np.uint8)
    sb = np.empty((rows // bm, cols // bn), np.uint8)
    nan = lib().orc_quant_fp4_block(_ptr(x), rows, cols, bm, bn, log2_kind, _ptr(packed), _ptr(sb))
    return packed, sb, nan


def dequant_fp8_block(codes, scale_f32, want_bf16=True):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    scale_f32 = np.ascontiguousarray(scale_f32, dtype=np.float32)
    rows, cols = codes.shape
    sr, sc = scale_f32.shape
    assert rows % sr == 0 and cols % sc == 0
    f = np.empty((rows, cols), np.float32)
    b = np.empty((rows, cols), np.uint16) if want_bf16 else None
    lib().orc_dequant_fp8_block(_ptr(codes), _ptr(scale_f32), rows, cols, rows // sr, cols // sc,
                                _ptr(f), _ptr(b) if want_bf16 else None)
    return f, b


def fp4_dequant(packed, scale_bytes, neg_zero, want_bf16=True):
    packed = np.ascontiguousarray(packed).view(np.uint8)
    scale_bytes = np.ascontiguousarray(scale_bytes).view(np.uint8)
    rows, half = packed.shape
    cols = half * 2
    sr, sc = scale_bytes.shape
    assert rows % sr == 0 and cols % sc == 0
    f = np.empty((rows, cols), np.float32)
    b = np.empty((rows, cols), np.uint16) if want_bf16 else None
    lib().orc_fp4_dequant(_ptr(packed), _ptr(scale_bytes), rows, cols, rows // sr, cols // sc,
                          neg_zero, _ptr(f), _ptr(b) if want_bf16 else None)
    return f, b


def fp4_to_e4m3_rebase(packed, scale_bytes):
    packed = np.ascontiguousarray(packed).view(np.uint8)
    scale_bytes = np.ascontiguousarray(scale_bytes).view(np.uint8)
    rows, half = packed.shape
    cols = half * 2
    assert rows % 128 == 0 and cols % 128 == 0 and scale_bytes.shape == (rows, cols // 32)
    q = np.empty((rows, cols), np.uint8)
    of = np.empty((rows // 128, cols // 128), np.float32)
    ob = np.empty((rows // 128, cols // 128), np.uint8)
    lib().orc_fp4_to_e4m3_rebase(_ptr(packed), _ptr(scale_bytes), rows, cols, _ptr(q), _ptr(of), _ptr(ob))
    return q, of, ob


def gemm_fp8_block(Aq, As, Bq, Bs):
    Aq = np.ascontiguousarray(Aq, dtype=np.uint8)
    Bq = np.ascontiguousarray(Bq, dtype=np.uint8)
    As = np.ascontiguousarray(As, dtype=np.float32)
    Bs = np.ascontiguousarray(Bs, dtype=np.float32)
    M, K = Aq.shape
    N = Bq.shape[0]
    C = np.empty((M, N), np.float32)
    lib().orc_gemm_fp8_block(_ptr(Aq), _ptr(As), _ptr(Bq), _ptr(Bs), M, N, K, _ptr(C))
    return C
