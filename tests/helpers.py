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
                ldx=None, ldy=None, mem=capi.MEM_DEVICE):
        """x: f32 [m, k] values; converted to the requested activation dtype before the call.  Device pointers by default (the
        kernels read the activations as they are); mem=MEM_HOST goes through the staged host path, which always scales the
        rows into the f16 range first."""
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
        if mem == capi.MEM_DEVICE and m > 0:
            xd, yd = self.dev_buffer(xsend), self.dev_buffer(y)
            bd = None if b is None else self.dev_buffer(b)
            try:
                capi.check(self.L.turq_qmatmul(self.ctx, w, xd, x_dtype, m, ldx, yd, y_dtype, ldy, bd, capi.MEM_DEVICE, algo), self.ctx)
                y = self.read_back(yd, (m, ldy), ydt)
            finally:
                for p in (xd, yd, bd):
                    if p is not None:
                        self.dev_free(p)
        else:
            capi.check(self.L.turq_qmatmul(self.ctx, w, capi.ptr(xsend), x_dtype, m, ldx, capi.ptr(y), y_dtype, ldy,
                                           capi.ptr(b), capi.MEM_HOST, algo), self.ctx)
        if y_dtype == capi.ACT_BF16:
            y = synth.from_bf16_bits(y).reshape(m, ldy)
        return np.asarray(y, np.float32)[:, :n]

    def dev_buffer(self, arr=None, nbytes=None):
        """device memory holding a copy of `arr` (or nbytes of uninitialised memory); free with dev_free"""
        p = ctypes.c_void_p()
        size = arr.nbytes if arr is not None else nbytes
        capi.check(self.L.turq_dev_alloc(self.ctx, max(size, 16), ctypes.byref(p)), self.ctx)
        if arr is not None:
            capi.check(self.L.turq_memcpy_h2d(self.ctx, p, capi.ptr(arr), arr.nbytes), self.ctx)
        return p

    def dev_free(self, p):
        capi.check(self.L.turq_dev_free(self.ctx, p), self.ctx)

    def read_back(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        capi.check(self.L.turq_memcpy_d2h(self.ctx, capi.ptr(out), p, out.nbytes), self.ctx)
        return out

    def qmatmul_device(self, w, x, n, k, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32, noalloc=False, algo=capi.ALGO_AUTO):
        """turq_qmatmul (or turq_qmatmul_noalloc) on device pointers; x: f32 values [m, k]; returns the output as the call
        wrote it (f32 values; bf16 outputs widened)"""
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        m = x.shape[0]
        xsend = (synth.to_bf16_bits(x).reshape(m, k) if x_dtype == capi.ACT_BF16 else x.astype(np.float16) if x_dtype == capi.ACT_F16 else x)
        ydt = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}[y_dtype]
        xd = self.dev_buffer(xsend)
        yd = self.dev_buffer(np.full((m, n), 0, ydt))
        try:
            if noalloc:
                rc = self.L.turq_qmatmul_noalloc(self.ctx, w, xd, x_dtype, m, k, yd, y_dtype, n, None)
            else:
                rc = self.L.turq_qmatmul(self.ctx, w, xd, x_dtype, m, k, yd, y_dtype, n, None, capi.MEM_DEVICE, algo)
            capi.check(rc, self.ctx)
            y = self.read_back(yd, (m, n), ydt)
        finally:
            self.dev_free(xd)
            self.dev_free(yd)
        if y_dtype == capi.ACT_BF16:
            y = synth.from_bf16_bits(y).reshape(m, n)
        return np.asarray(y, np.float32)

    def qmatmul_multi(self, ws, x, ns, k, x_dtype=capi.ACT_F32, biases=None, mem=capi.MEM_DEVICE):
        """several weights against the same activations through turq_qmatmul_multi; f32 outputs.
        With mem = MEM_DEVICE the activations, biases and outputs live in device buffers."""
        L, ctx = self.L, self.ctx
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        m = x.shape[0]
        xsend = synth.to_bf16_bits(x).reshape(m, k) if x_dtype == capi.ACT_BF16 else x.astype(np.float16) if x_dtype == capi.ACT_F16 else x
        count = len(ws)
        outs = [np.zeros((m, n), np.float32) for n in ns]
        bias_host = [None if biases is None or b is None else np.ascontiguousarray(b, np.float32) for b in (biases or [None] * count)]
        freed = []

        def dev(nbytes):
            p = ctypes.c_void_p()
            capi.check(L.turq_dev_alloc(ctx, max(nbytes, 16), ctypes.byref(p)), ctx)
            freed.append(p)
            return p

        if mem == capi.MEM_DEVICE:
            xd = dev(xsend.nbytes)
            capi.check(L.turq_memcpy_h2d(ctx, xd, capi.ptr(xsend), xsend.nbytes), ctx)
            yd = [dev(o.nbytes) for o in outs]
            bd = []
            for b in bias_host:
                if b is None:
                    bd.append(None)
                else:
                    p = dev(b.nbytes)
                    capi.check(L.turq_memcpy_h2d(ctx, p, capi.ptr(b), b.nbytes), ctx)
                    bd.append(p)
            xp, yp, bp = xd, [p.value for p in yd], [None if p is None else p.value for p in bd]
        else:
            xp, yp = capi.ptr(xsend), [o.ctypes.data for o in outs]
            bp = [None if b is None else b.ctypes.data for b in bias_host]
        warr = (ctypes.c_void_p * count)(*[w.value for w in ws])
        yarr = (ctypes.c_void_p * count)(*yp)
        barr = (ctypes.c_void_p * count)(*bp)
        ldys = (ctypes.c_int64 * count)(*ns)
        rc = L.turq_qmatmul_multi(ctx, count, warr, xp, x_dtype, m, k, yarr, capi.ACT_F32, ldys,
                                  barr if biases is not None else None, mem, capi.ALGO_AUTO)
        capi.check(rc, ctx)
        if mem == capi.MEM_DEVICE:
            for o, p in zip(outs, yd):
                capi.check(L.turq_memcpy_d2h(ctx, capi.ptr(o), p, o.nbytes), ctx)
        for p in freed:
            capi.check(L.turq_dev_free(ctx, p), ctx)
        return outs

    def gate_up(self, wg, wu, x, n, k, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32, bias_gate=None, bias_up=None,
                mem=capi.MEM_DEVICE, ldx=None, ldy=None):
        """act(x gate^T) * (x up^T) through turq_qmatmul_gate_up; returns f32 [m, n]"""
        L, ctx = self.L, self.ctx
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        m = x.shape[0]
        ldx, ldy = ldx or k, ldy or n
        xbuf = np.zeros((m, ldx), np.float32)
        xbuf[:, :k] = x
        xsend = (synth.to_bf16_bits(xbuf).reshape(m, ldx) if x_dtype == capi.ACT_BF16
                 else xbuf.astype(np.float16) if x_dtype == capi.ACT_F16 else xbuf)
        ydt = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}[y_dtype]
        y = np.full((m, ldy), 0, ydt)
        bg = None if bias_gate is None else np.ascontiguousarray(bias_gate, np.float32)
        bu = None if bias_up is None else np.ascontiguousarray(bias_up, np.float32)
        freed = []

        def dev(arr):
            p = ctypes.c_void_p()
            capi.check(L.turq_dev_alloc(ctx, max(arr.nbytes, 16), ctypes.byref(p)), ctx)
            freed.append(p)
            capi.check(L.turq_memcpy_h2d(ctx, p, capi.ptr(arr), arr.nbytes), ctx)
            return p

        if mem == capi.MEM_DEVICE:
            xp, yp = dev(xsend), dev(y)
            bgp = None if bg is None else dev(bg)
            bup = None if bu is None else dev(bu)
        else:
            xp, yp, bgp, bup = capi.ptr(xsend), capi.ptr(y), capi.ptr(bg), capi.ptr(bu)
        rc = L.turq_qmatmul_gate_up(ctx, wg, wu, xp, x_dtype, m, ldx, yp, y_dtype, ldy, bgp, bup, 0, mem)
        capi.check(rc, ctx)
        if mem == capi.MEM_DEVICE:
            capi.check(L.turq_memcpy_d2h(ctx, capi.ptr(y), yp, y.nbytes), ctx)
        for p in freed:
            capi.check(L.turq_dev_free(ctx, p), ctx)
        if y_dtype == capi.ACT_BF16:
            y = synth.from_bf16_bits(y).reshape(m, ldy)
        return np.asarray(y, np.float32)[:, :n]

    def mlp(self, wg, wu, wd, x, n_ff, k, n_out, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32, biases=(None, None, None),
            mem=capi.MEM_DEVICE, launches=None):
        """down(act(gate(x)) * up(x)) through turq_mlp; returns f32 [m, n_out].  launches: a list that receives the number of
        matmul kernel launches the call made (device pointers only; from the library's kernel timing)."""
        L, ctx = self.L, self.ctx
        x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
        m = x.shape[0]
        xsend = (synth.to_bf16_bits(x).reshape(m, k) if x_dtype == capi.ACT_BF16 else x.astype(np.float16) if x_dtype == capi.ACT_F16 else x)
        ydt = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}[y_dtype]
        y = np.full((m, n_out), 0, ydt)
        bs = [None if b is None else np.ascontiguousarray(b, np.float32) for b in biases]
        freed = []
        if mem == capi.MEM_DEVICE:
            def dev(arr):
                p = self.dev_buffer(arr)
                freed.append(p)
                return p
            xp, yp = dev(xsend), dev(y)
            bp = [None if b is None else dev(b) for b in bs]
        else:
            xp, yp, bp = capi.ptr(xsend), capi.ptr(y), [capi.ptr(b) for b in bs]
        try:
            if launches is not None:
                capi.check(L.turq_profile_begin(ctx), ctx)
            rc = L.turq_mlp(ctx, wg, wu, wd, xp, x_dtype, m, k, yp, y_dtype, n_out, bp[0], bp[1], bp[2], 0, mem)
            if launches is not None:
                cnt, ms = ctypes.c_int64(), ctypes.c_double()
                capi.check(L.turq_profile_end(ctx, ctypes.byref(cnt), ctypes.byref(ms)), ctx)
                launches.append(cnt.value)
            capi.check(rc, ctx)
            capi.check(L.turq_sync(ctx), ctx)
            if mem == capi.MEM_DEVICE:
                y = self.read_back(yp, (m, n_out), ydt)
        finally:
            for p in freed:
                self.dev_free(p)
        if y_dtype == capi.ACT_BF16:
            y = synth.from_bf16_bits(y).reshape(m, n_out)
        return np.asarray(y, np.float32)

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
