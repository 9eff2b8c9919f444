"""ctypes loader for the CPU oracle (``libopencnn_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``; never by the ``opencnn_amd`` package.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libopencnn_oracle.so")

_fp = ctypes.POINTER(ctypes.c_float)
_dp = ctypes.POINTER(ctypes.c_double)
_i = ctypes.c_int
_lib = None


def build() -> None:
    subprocess.run(["make", "-C", _HERE, "-B", "libopencnn_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        h = ctypes.CDLL(LIB_PATH)
        h.oracle_num_threads.restype = _i
        h.oracle_tiles_dim.restype = _i
        h.oracle_tiles_dim.argtypes = [_i]
        h.oracle_direct_conv_f64.restype = None
        h.oracle_direct_conv_f64.argtypes = [_fp, _fp, _dp, _i, _i, _i, _i, _i]
        h.oracle_fx.restype = None
        h.oracle_fx.argtypes = [_fp, _fp, _i, _i]
        h.oracle_fx_one.restype = None
        h.oracle_fx_one.argtypes = [_fp, _fp]
        h.oracle_input_transform.restype = None
        h.oracle_input_transform.argtypes = [_fp, _fp]
        h.oracle_output_transform.restype = None
        h.oracle_output_transform.argtypes = [_fp, _fp]
        h.oracle_round_operand.restype = ctypes.c_float
        h.oracle_round_operand.argtypes = [ctypes.c_float, _i]
        h.oracle_winograd_f32.restype = _i
        h.oracle_winograd_f32.argtypes = [_fp, _fp, _fp, _i, _i, _i, _i, _i, _i]
        for name, want in (("oracle_compare_f32_f64", _dp), ("oracle_compare_f32_f32", _fp)):
            f = getattr(h, name)
            f.restype = None
            f.argtypes = [_fp, want, ctypes.c_long, _dp, _dp, _dp]
        _lib = h
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t=_fp):
    return a.ctypes.data_as(t)


def num_threads() -> int:
    return lib().oracle_num_threads()


def tiles_dim(in_w: int) -> int:
    return lib().oracle_tiles_dim(in_w)


def direct_conv_f64(x_chwn, w_crsk) -> np.ndarray:
    """fp64 direct cross-correlation, pad 1, stride 1: CHWN, CRSK -> KHWN (float64)."""
    x, w = _f32(x_chwn), _f32(w_crsk)
    C, H, W, N = x.shape
    K = w.shape[3]
    assert w.shape == (C, 3, 3, K)
    y = np.empty((K, H, W, N), dtype=np.float64)
    lib().oracle_direct_conv_f64(_p(x), _p(w), _p(y, _dp), N, C, H, W, K)
    return y


def fx(w_crsk) -> np.ndarray:
    """CRSK -> [C][16][K] in the reference's arithmetic order."""
    w = _f32(w_crsk)
    C, _, _, K = w.shape
    out = np.empty((C, 16, K), dtype=np.float32)
    lib().oracle_fx(_p(w), _p(out), C, K)
    return out


def fx_one(g9) -> np.ndarray:
    g = _f32(g9).reshape(9)
    out = np.empty(16, dtype=np.float32)
    lib().oracle_fx_one(_p(g), _p(out))
    return out


def input_transform(d16) -> np.ndarray:
    d = _f32(d16).reshape(16)
    out = np.empty(16, dtype=np.float32)
    lib().oracle_input_transform(_p(d), _p(out))
    return out


def output_transform(m16) -> np.ndarray:
    m = _f32(m16).reshape(16)
    out = np.empty(4, dtype=np.float32)
    lib().oracle_output_transform(_p(m), _p(out))
    return out


def round_operand(v: float, quant: int) -> float:
    return float(lib().oracle_round_operand(float(v), quant))


def winograd_f32(x_chwn, w_crsk, quant: int = 0) -> np.ndarray:
    """The whole path in the reference's order; quant 0 fp32, 1 fp16, 2 bf16 operands."""
    x, w = _f32(x_chwn), _f32(w_crsk)
    C, H, W, N = x.shape
    K = w.shape[3]
    assert w.shape == (C, 3, 3, K)
    y = np.full((K, H, W, N), np.nan, dtype=np.float32)
    rc = lib().oracle_winograd_f32(_p(x), _p(w), _p(y), N, C, H, W, K, quant)
    if rc != 0:
        raise ValueError("oracle_winograd_f32 does not model this shape")
    return y


def compare(got, want):
    """(rel_l2, max_abs, max_ref) of got (float32) against want (float32 or float64)."""
    g = _f32(got)
    rel, ma, mr = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    if want.dtype == np.float64:
        w = np.ascontiguousarray(want)
        lib().oracle_compare_f32_f64(_p(g), _p(w, _dp), g.size, rel, ma, mr)
    else:
        w = _f32(want)
        lib().oracle_compare_f32_f32(_p(g), _p(w), g.size, rel, ma, mr)
    assert g.size == w.size
    return rel.value, ma.value, mr.value
