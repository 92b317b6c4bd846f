"""TEST INFRASTRUCTURE ONLY — ctypes binding of ``oracle/twl_oracle.c``.

Each wrapper cites the reference lines the C function restates; see the header of
``twl_oracle.c`` for how every function is pinned.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtwl_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``twl_oracle.c`` with gcc (through the Makefile beside it)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libtwl_oracle.so"], check=True, capture_output=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        src = os.path.join(_HERE, "twl_oracle.c")
        if not os.path.exists(_SO) or (
            os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_SO)
        ):
            build()
        L = ctypes.CDLL(_SO)
        u8p = ctypes.POINTER(ctypes.c_uint8)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        f32p = ctypes.POINTER(ctypes.c_float)
        i32p = ctypes.POINTER(ctypes.c_int32)
        L.twl_oracle_top_p_f32.argtypes = [f32p, u8p, f32p, ctypes.c_float, ctypes.c_uint32,
                                           ctypes.c_uint32, ctypes.c_int, f32p, i32p, f32p]
        L.twl_oracle_top_p_f32.restype = None
        L.twl_oracle_top_p_cub.argtypes = [ctypes.c_void_p, ctypes.c_int, u8p, f32p, ctypes.c_float,
                                           ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int, f32p, i32p]
        L.twl_oracle_top_p_cub.restype = None
        L.twl_oracle_dt_add.argtypes = [ctypes.c_double, ctypes.c_double, ctypes.c_int]
        L.twl_oracle_dt_add.restype = ctypes.c_double
        L.twl_oracle_dt_round.argtypes = [ctypes.c_double, ctypes.c_int]
        L.twl_oracle_dt_round.restype = ctypes.c_double
        L.twl_oracle_nucleus.argtypes = [f32p, ctypes.c_uint32, ctypes.c_double, u8p, f32p,
                                         ctypes.POINTER(ctypes.c_double)]
        L.twl_oracle_nucleus.restype = ctypes.c_uint32
        L.twl_oracle_int4_quant.argtypes = [f32p, ctypes.c_uint32, ctypes.c_uint32, u8p, u16p, u16p]
        L.twl_oracle_int4_quant.restype = None
        L.twl_oracle_int4_dequant.argtypes = [u8p, u16p, u16p, ctypes.c_uint32, ctypes.c_uint32, f32p]
        L.twl_oracle_int4_dequant.restype = None
        L.twl_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.twl_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.twl_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.twl_oracle_f16_to_f32.restype = ctypes.c_float
        L.twl_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.twl_oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib = L
    return _lib


def _ptr(a: np.ndarray, ctype):
    return a.ctypes.data_as(ctypes.POINTER(ctype))


HIGH_FIRST = 0  # csrc/include/sampling.cuh:156-159 as written
HIGH_MAX = 1    # paper Algorithm 1


def top_p_mask_f32(probs: np.ndarray, p, high_mode: int = HIGH_FIRST, return_margin: bool = False):
    """csrc/include/sampling.cuh:156-231 on a [rows, d] fp32 array.

    ``p`` is a float or a per-row array (``top_p_arr``, sampling.cuh:125).
    Returns ``(mask uint8 [rows,d], low float32 [rows], iters int32 [rows])``; with
    ``return_margin`` also the smallest ``|S - p|`` met per row (a decision with a margin of a few
    fp32 ulps may flip under another summation order).
    """
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    assert probs.ndim == 2
    rows, d = probs.shape
    mask = np.zeros((rows, d), dtype=np.uint8)
    low = np.zeros(rows, dtype=np.float32)
    iters = np.zeros(rows, dtype=np.int32)
    margin = np.zeros(rows, dtype=np.float32)
    if isinstance(p, np.ndarray):
        p_arr = np.ascontiguousarray(p, dtype=np.float32)
        assert p_arr.shape == (rows,)
        pp, pv = _ptr(p_arr, ctypes.c_float), 0.0
    else:
        pp, pv = None, float(p)
    lib().twl_oracle_top_p_f32(_ptr(probs, ctypes.c_float), _ptr(mask, ctypes.c_uint8), pp, pv,
                               rows, d, int(high_mode), _ptr(low, ctypes.c_float),
                               _ptr(iters, ctypes.c_int32), _ptr(margin, ctypes.c_float))
    if return_margin:
        return mask, low, iters, margin
    return mask, low, iters


DT_F16, DT_BF16, DT_F32 = 0, 1, 2


def top_p_mask_cub(values: np.ndarray, dtype: int, p, high_mode: int = HIGH_FIRST):
    """``TopPReturnMaskKernel`` with every operation in its element type and the additions in the
    order of ``cub::BlockReduce`` (csrc/include/sampling.cuh:54,119-231; csrc/src/sampling.cu:22-63).

    ``values`` [rows, d]: the uint16 view of fp16 (``dtype`` 0) or bf16 (1) probabilities, or
    float32 (2). Returns ``(mask uint8 [rows,d], low float32 [rows], iters int32 [rows])``; for
    this function the result is exact, there is no margin.
    """
    values = np.ascontiguousarray(values, dtype=np.float32 if dtype == DT_F32 else np.uint16)
    rows, d = values.shape
    mask = np.zeros((rows, d), dtype=np.uint8)
    low = np.zeros(rows, dtype=np.float32)
    iters = np.zeros(rows, dtype=np.int32)
    if isinstance(p, np.ndarray):
        p_arr = np.ascontiguousarray(p, dtype=np.float32)
        pp, pv = _ptr(p_arr, ctypes.c_float), 0.0
    else:
        pp, pv = None, float(p)
    lib().twl_oracle_top_p_cub(values.ctypes.data_as(ctypes.c_void_p), int(dtype),
                               _ptr(mask, ctypes.c_uint8), pp, pv, rows, d, int(high_mode),
                               _ptr(low, ctypes.c_float), _ptr(iters, ctypes.c_int32))
    return mask, low, iters


def dt_add(a: float, b: float, dtype: int) -> float:
    """One addition in the element type (round to nearest even), as the oracle performs it."""
    return float(lib().twl_oracle_dt_add(float(a), float(b), int(dtype)))


def dt_round(x: float, dtype: int) -> float:
    return float(lib().twl_oracle_dt_round(float(x), int(dtype)))


def nucleus(probs_row: np.ndarray, p: float):
    """Textbook minimal top-p set of one row (ties with the pivot kept): ``(mask, pivot, mass)``."""
    x = np.ascontiguousarray(probs_row, dtype=np.float32)
    assert x.ndim == 1
    mask = np.zeros(x.shape[0], dtype=np.uint8)
    pivot = ctypes.c_float(0)
    mass = ctypes.c_double(0)
    lib().twl_oracle_nucleus(_ptr(x, ctypes.c_float), x.shape[0], float(p),
                             _ptr(mask, ctypes.c_uint8), ctypes.byref(pivot), ctypes.byref(mass))
    return mask, float(pivot.value), float(mass.value)


def int4_quant(k: np.ndarray, group: int = 32):
    """twilight/pyimpl/quantize.py:4-13 per group of ``group`` with fp16 scale/zero storage.

    ``k`` [..., D] fp32 -> ``(codes uint8 [..., D], scale float16 [..., D/group], zero float16 [...])``.
    """
    k = np.ascontiguousarray(k, dtype=np.float32)
    D = k.shape[-1]
    assert D % group == 0
    n_groups = k.size // group
    codes = np.zeros(k.shape, dtype=np.uint8)
    gshape = k.shape[:-1] + (D // group,)
    scale = np.zeros(gshape, dtype=np.uint16)
    zero = np.zeros(gshape, dtype=np.uint16)
    lib().twl_oracle_int4_quant(_ptr(k, ctypes.c_float), n_groups, group,
                                _ptr(codes, ctypes.c_uint8), _ptr(scale, ctypes.c_uint16),
                                _ptr(zero, ctypes.c_uint16))
    return codes, scale.view(np.float16), zero.view(np.float16)


def int4_dequant(codes: np.ndarray, scale: np.ndarray, zero: np.ndarray, group: int = 32):
    """``float(code) * float(scale) + float(zero)`` with one fp32 rounding -> fp32 [..., D]."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    scale = np.ascontiguousarray(scale, dtype=np.float16)
    zero = np.ascontiguousarray(zero, dtype=np.float16)
    out = np.zeros(codes.shape, dtype=np.float32)
    lib().twl_oracle_int4_dequant(_ptr(codes, ctypes.c_uint8),
                                  _ptr(scale.view(np.uint16), ctypes.c_uint16),
                                  _ptr(zero.view(np.uint16), ctypes.c_uint16),
                                  codes.size // group, group, _ptr(out, ctypes.c_float))
    return out
