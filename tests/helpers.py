"""Shared helpers of the GPU parity tests: a context, weight upload and calls through the C ABI."""
from __future__ import annotations

import ctypes

import numpy as np

from tur_amd import capi, synth


class Gpu:
    """One libturq context; every call goes through the C ABI."""

    def __init__(self, device: int = 0):
        self.L = capi.lib()
        h = ctypes.c_void_p()
        capi.check(self.L.turq_ctx_create(device, ctypes.byref(h)))
        self.ctx = h

    def close(self):
        if self.ctx:
            self.L.turq_ctx_destroy(self.ctx)
            self.ctx = None

    def upload(self, dt, n, k, raw, layout):
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        w = ctypes.c_void_p()
        capi.check(self.L.turq_weight_upload(self.ctx, dt, n, k, capi.ptr(raw), raw.size, layout, ctypes.byref(w)), self.ctx)
        return w

    def release(self, w):
        capi.check(self.L.turq_weight_release(w))

    def dequantize(self, w, n, k):
        out = np.empty(n * k, np.float32)
        capi.check(self.L.turq_dequantize(self.ctx, w, capi.ptr(out), capi.MEM_HOST), self.ctx)
        return out

    def export(self, w, nbytes):
        out = np.empty(nbytes, np.uint8)
        capi.check(self.L.turq_weight_export(self.ctx, w, capi.ptr(out), nbytes), self.ctx)
        return out

    def qmatmul(self, w, x, n, k, algo=capi.ALGO_AUTO, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32, bias=None,
                ldx=None, ldy=None):
        """x: f32 [m, k] values; converted to the requested activation dtype before the call."""
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        m = x.shape[0]
        ldx = ldx or k
        ldy = ldy or n
        xbuf = np.zeros((m, ldx), np.float32)
        xbuf[:, :k] = x
        if x_dtype == capi.ACT_BF16:
            xsend = synth.to_bf16_bits(xbuf).reshape(m, ldx)
        elif x_dtype == capi.ACT_F16:
            xsend = xbuf.astype(np.float16)
        else:
            xsend = xbuf
        ydt = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}[y_dtype]
        y = np.zeros((m, ldy), ydt)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        capi.check(self.L.turq_qmatmul(self.ctx, w, capi.ptr(xsend), x_dtype, m, ldx, capi.ptr(y), y_dtype, ldy,
                                       capi.ptr(b), capi.MEM_HOST, algo), self.ctx)
        if y_dtype == capi.ACT_BF16:
            y = synth.from_bf16_bits(y).reshape(m, ldy)
        return np.asarray(y, np.float32)[:, :n]

    def quantize(self, x, kind):
        x = np.ascontiguousarray(x, np.float32)
        m, k = x.shape
        if kind == "q8_0":
            out = np.zeros((m * k // 32, 34), np.uint8)
            capi.check(self.L.turq_quantize_q8_0(self.ctx, capi.ptr(x), m, k, capi.ptr(out), capi.MEM_HOST), self.ctx)
        else:
            out = np.zeros((m * k // 256, 292), np.uint8)
            capi.check(self.L.turq_quantize_q8_k(self.ctx, capi.ptr(x), m, k, capi.ptr(out), capi.MEM_HOST), self.ctx)
        return out


def rel_l2(a, b) -> float:
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
