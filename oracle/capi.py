"""ctypes access to ``libturq_oracle.so`` (the plain-C restatement in ``turq_oracle.c``).

Test infrastructure: imported by ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s
``cpu_baseline`` leg only.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libturq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libturq_oracle.so"])
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_bf16_to_f32.restype = ctypes.c_float
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_block_elems.argtypes = [ci]
        L.orc_block_bytes.argtypes = [ci]
        L.orc_dequantize.argtypes = [ci, vp, i64, vp]
        L.orc_quantize_q8_0.argtypes = [vp, i64, vp]
        L.orc_quantize_q8_K.argtypes = [vp, i64, vp]
        L.orc_vec_dot.restype = ctypes.c_float
        L.orc_vec_dot.argtypes = [ci, i64, vp, vp]
        L.orc_qmatmul.argtypes = [ci, i64, i64, i64, vp, vp, vp, ci]
        L.orc_matmul_dequant.argtypes = [ci, i64, i64, i64, vp, vp, vp, ci]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def dequantize(dtype: int, raw: np.ndarray) -> np.ndarray:
    L = lib()
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    nelem = raw.size // L.orc_block_bytes(dtype) * L.orc_block_elems(dtype)
    out = np.empty(nelem, np.float32)
    if L.orc_dequantize(dtype, _p(raw), nelem, _p(out)) != 0:
        raise ValueError("orc_dequantize failed")
    return out


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    out = np.zeros((x.size // 32, 34), np.uint8)
    if lib().orc_quantize_q8_0(_p(x), x.size, _p(out)) != 0:
        raise ValueError("k must be a multiple of 32")
    return out


def quantize_q8_K(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    out = np.zeros((x.size // 256, 292), np.uint8)
    if lib().orc_quantize_q8_K(_p(x), x.size, _p(out)) != 0:
        raise ValueError("k must be a multiple of 256")
    return out


def qmatmul(dtype: int, x: np.ndarray, raw: np.ndarray, n: int, k: int, nthreads: int = 0) -> np.ndarray:
    """restated candle CPU QMatMul::forward (quantises the activations)"""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    out = np.empty((x.shape[0], n), np.float32)
    nt = nthreads or (os.cpu_count() or 1)
    if lib().orc_qmatmul(dtype, x.shape[0], k, n, _p(x), _p(raw), _p(out), nt) != 0:
        raise ValueError("orc_qmatmul failed")
    return out


def matmul_dequant(dtype: int, x: np.ndarray, raw: np.ndarray, n: int, k: int, nthreads: int = 0) -> np.ndarray:
    """x @ dequantize(W).T with f64 accumulation"""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    out = np.empty((x.shape[0], n), np.float32)
    nt = nthreads or (os.cpu_count() or 1)
    if lib().orc_matmul_dequant(dtype, x.shape[0], k, n, _p(x), _p(raw), _p(out), nt) != 0:
        raise ValueError("orc_matmul_dequant failed")
    return out
