"""Host-side mirror of the reference's quantized-linear interface, on top of the C ABI.

Same names, argument meaning and error behaviour as the reference so that tests read like its own:

* ``Device``          — the ``candle_core::Device`` handed to ``QVarBuilder::from_gguf`` (a libturq context);
* ``QTensor``         — ``candle_core::quantized::QTensor``: raw blocks on the device, ``shape()``, ``dtype()``,
                        ``dequantize()``; clones share one device copy (``Arc<QTensor>``);
* ``QMatMul``         — ``QMatMul::from_arc(qtensor)`` + ``forward(x)``;
* ``LinearX``         — ``src/models/layers/linear.rs:8-31``: ``Quantized{qmatmul, bias}``, ``forward`` adds the bias;
* ``QVarBuilder``     — ``src/weights/gguf_varbuilder.rs``: ``from_gguf``, ``pp``, ``get``, ``get_no_shape``,
                        ``contains_key``, ``tensor_shape``, ``all_keys``, with the one-entry last-tensor cache;
* ``linear(in_dim, out_dim, vb)`` — ``src/models/layers/linear.rs:50-70`` (GGUF arm);
* ``NormX`` / ``rms_norm(size, eps, vb)`` — ``src/models/layers/norm.rs:9-94`` (GGUF arm, RmsNorm).

Activations and results are NumPy arrays on the host here (this mirror is for tests and scripting; an engine
binds the C ABI directly and keeps its tensors on the device).
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import capi, synth
from .capi import TurqError


class Device:
    """One GPU context (device ordinal + stream + scratch)."""

    def __init__(self, ordinal: int = 0):
        self.L = capi.lib()
        h = ctypes.c_void_p()
        capi.check(self.L.turq_ctx_create(ordinal, ctypes.byref(h)))
        self.ctx = h
        self.ordinal = ordinal

    @staticmethod
    def new_hip(ordinal: int = 0) -> "Device":
        return Device(ordinal)

    def nonfinite_count(self, reset: bool = True) -> int:
        """results stored since the last reset that were no finite numbers (``turq_ctx_nonfinite_count``)"""
        import ctypes

        n = ctypes.c_uint64()
        capi.check(self.L.turq_ctx_nonfinite_count(self.ctx, ctypes.byref(n), 1 if reset else 0), self.ctx)
        return n.value

    def synchronize(self) -> None:
        capi.check(self.L.turq_sync(self.ctx), self.ctx)

    def close(self) -> None:
        if self.ctx:
            self.L.turq_ctx_destroy(self.ctx)
            self.ctx = None


class QTensor:
    """Quantized (or dense F32/F16/BF16) GGUF tensor resident in HBM."""

    def __init__(self, device: Device, handle, owns: bool = True):
        self.device = device
        self.handle = handle
        self._owns = owns
        dt, n, k, layout, nbytes = ctypes.c_int(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int(), ctypes.c_size_t()
        capi.check(device.L.turq_weight_info(handle, ctypes.byref(dt), ctypes.byref(n), ctypes.byref(k), ctypes.byref(layout),
                                             ctypes.byref(nbytes)))
        self._dtype, self._n, self._k, self._layout, self._nbytes = dt.value, n.value, k.value, layout.value, nbytes.value
        self._one_dim = False

    @classmethod
    def new(cls, device: Device, ggml_dtype: int, shape: Sequence[int], raw, layout: int = capi.LAYOUT_TILED) -> "QTensor":
        """raw GGUF block bytes of a tensor of ``shape`` = (n, k) or (k,)"""
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        n, k = (1, shape[0]) if len(shape) == 1 else (shape[0], shape[1])
        if not (ggml_dtype in (capi.Q8_0, capi.Q4_K, capi.Q5_K, capi.Q6_K)):
            layout = capi.LAYOUT_NATIVE
        h = ctypes.c_void_p()
        capi.check(device.L.turq_weight_upload(device.ctx, ggml_dtype, n, k, capi.ptr(raw), raw.size, layout, ctypes.byref(h)),
                   device.ctx)
        t = cls(device, h)
        t._one_dim = len(shape) == 1
        return t

    def shape(self) -> Tuple[int, ...]:
        return (self._k,) if self._one_dim else (self._n, self._k)

    def dtype(self) -> int:
        return self._dtype

    def clone(self) -> "QTensor":
        capi.check(self.device.L.turq_weight_retain(self.handle))
        t = QTensor(self.device, self.handle)
        t._one_dim = self._one_dim
        return t

    def dequantize(self, device: Optional[Device] = None) -> np.ndarray:
        """f32 array of ``shape()`` — bit-exact with candle's ``QTensor::dequantize``"""
        dev = device or self.device
        out = np.empty(self._n * self._k, np.float32)
        capi.check(dev.L.turq_dequantize(dev.ctx, self.handle, capi.ptr(out), capi.MEM_HOST), dev.ctx)
        return out.reshape(self.shape())

    def release(self) -> None:
        if self._owns and self.handle:
            self.device.L.turq_weight_release(self.handle)
            self.handle = None

    def __del__(self):  # Arc drop
        try:
            self.release()
        except Exception:
            pass


def dequantize_all() -> bool:
    """candle's switch: with CANDLE_DEQUANTIZE_ALL (or CANDLE_DEQUANTIZE_ALL_F16) set, ``QMatMul::from_arc`` turns every
    tensor into a dense matmul instead of the quantized one"""
    import os

    return bool(os.environ.get("CANDLE_DEQUANTIZE_ALL") or os.environ.get("CANDLE_DEQUANTIZE_ALL_F16"))


class QMatMul:
    """``QMatMul::from_arc`` + ``forward``: y = x @ W.T for x of shape [..., k].

    As in candle, a block-quantized tensor gives the quantized matmul (``QMatMul::QTensor``) and an F32 / F16 / BF16 tensor -
    or any tensor while ``CANDLE_DEQUANTIZE_ALL`` is set - the dense one (``QMatMul::Tensor``): f32 arithmetic on the
    dequantized weights, activations not rounded (here: the plain kernel on the tensor's GGUF bytes, which dequantizes on
    the fly; a tiled tensor is re-uploaded in GGUF order for it)."""

    def __init__(self, qtensor: QTensor, dense: Optional[bool] = None):
        quant = qtensor.dtype() in (capi.Q8_0, capi.Q4_K, capi.Q5_K, capi.Q6_K)
        if not quant and qtensor.dtype() not in (capi.F32, capi.F16, capi.BF16):
            raise TurqError(capi.ERR_DTYPE, f"QMatMul: unsupported ggml dtype {qtensor.dtype()}")
        self.dense = (not quant) or (dequantize_all() if dense is None else dense)
        if self.dense and qtensor._layout != capi.LAYOUT_NATIVE:
            dev = qtensor.device
            raw = np.empty(synth.weight_nbytes(qtensor.dtype(), qtensor._n, qtensor._k), np.uint8)
            capi.check(dev.L.turq_weight_export(dev.ctx, qtensor.handle, capi.ptr(raw), raw.size), dev.ctx)
            qtensor = QTensor.new(dev, qtensor.dtype(), (qtensor._n, qtensor._k), raw, capi.LAYOUT_NATIVE)
        self.qtensor = qtensor

    @classmethod
    def from_arc(cls, qtensor: QTensor) -> "QMatMul":
        return cls(qtensor)

    def forward(self, xs: np.ndarray, bias: Optional[np.ndarray] = None, algo: int = capi.ALGO_AUTO) -> np.ndarray:
        q = self.qtensor
        n, k = q._n, q._k
        xs = np.asarray(xs)
        if xs.ndim < 2:
            raise TurqError(capi.ERR_SHAPE, f"QMatMul::forward needs rank >= 2, got shape {xs.shape}")
        if xs.shape[-1] != k:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: last dim {xs.shape[-1]} != {k}")
        if xs.dtype == np.float32:
            xt = capi.ACT_F32
        elif xs.dtype == np.float16:
            xt = capi.ACT_F16
        else:
            raise TurqError(capi.ERR_DTYPE, f"unsupported activation dtype {xs.dtype}")
        if not xs.flags["C_CONTIGUOUS"]:
            raise TurqError(capi.ERR_INVALID, "QMatMul::forward needs a contiguous input")
        lead = xs.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        y = np.empty((m, n), np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        dev = q.device
        if self.dense:
            algo = capi.ALGO_SIMPLE
        capi.check(dev.L.turq_qmatmul(dev.ctx, q.handle, capi.ptr(xs), xt, m, k, capi.ptr(y), capi.ACT_F32, n, capi.ptr(b),
                                      capi.MEM_HOST, algo), dev.ctx)
        return y.reshape(lead + (n,))

    @staticmethod
    def forward_multi(layers: "list[QMatMul]", xs: np.ndarray, biases: "Optional[list]" = None) -> "list[np.ndarray]":
        """Several projections of one tensor (q / k / v, gate / up: src/models/qwen3.rs:161-167, 272-274) through
        ``turq_qmatmul_multi``.  With host arrays, as here, that is the single calls one after the other; with
        device-resident activations and up to four rows it is one kernel launch per run of equal formats."""
        import ctypes

        if not layers:
            return []
        xs = np.asarray(xs)
        k = layers[0].qtensor._k
        if xs.ndim < 2 or xs.shape[-1] != k or any(l.qtensor._k != k for l in layers):
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: input {xs.shape}, layers need last dim {k}")
        if xs.dtype != np.float32 or not xs.flags["C_CONTIGUOUS"]:
            raise TurqError(capi.ERR_INVALID, "forward_multi needs a contiguous f32 input")
        lead = xs.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        cnt = len(layers)
        ys = [np.empty((m, l.qtensor._n), np.float32) for l in layers]
        bs = [None if biases is None or b is None else np.ascontiguousarray(b, np.float32) for b in (biases or [None] * cnt)]
        warr = (ctypes.c_void_p * cnt)(*[l.qtensor.handle.value for l in layers])
        yarr = (ctypes.c_void_p * cnt)(*[y.ctypes.data for y in ys])
        barr = (ctypes.c_void_p * cnt)(*[None if b is None else b.ctypes.data for b in bs])
        ldys = (ctypes.c_int64 * cnt)(*[l.qtensor._n for l in layers])
        dev = layers[0].qtensor.device
        capi.check(dev.L.turq_qmatmul_multi(dev.ctx, cnt, warr, capi.ptr(xs), capi.ACT_F32, m, k, yarr, capi.ACT_F32, ldys,
                                            barr if biases is not None else None, capi.MEM_HOST, capi.ALGO_AUTO), dev.ctx)
        return [y.reshape(lead + (y.shape[1],)) for y in ys]


    @staticmethod
    def forward_gate_up(gate: "QMatMul", up: "QMatMul", xs: np.ndarray, bias_gate: Optional[np.ndarray] = None,
                        bias_up: Optional[np.ndarray] = None) -> np.ndarray:
        """``silu(x @ gate.T) * (x @ up.T)``, the first half of ``Qwen3MLP::forward`` (src/models/qwen3.rs:161-167), through
        ``turq_qmatmul_gate_up``.  With host arrays, as here, the two products go through the host path and are combined on the
        host; with device-resident activations and one or two rows it is one kernel launch that writes the product."""
        xs = np.asarray(xs)
        n, k = gate.qtensor._n, gate.qtensor._k
        if xs.ndim < 2 or xs.shape[-1] != k:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: input {xs.shape}, layers need last dim {k}")
        if xs.dtype != np.float32 or not xs.flags["C_CONTIGUOUS"]:
            raise TurqError(capi.ERR_INVALID, "forward_gate_up needs a contiguous f32 input")
        lead = xs.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        y = np.empty((m, n), np.float32)
        bg = None if bias_gate is None else np.ascontiguousarray(bias_gate, np.float32)
        bu = None if bias_up is None else np.ascontiguousarray(bias_up, np.float32)
        dev = gate.qtensor.device
        capi.check(dev.L.turq_qmatmul_gate_up(dev.ctx, gate.qtensor.handle, up.qtensor.handle, capi.ptr(xs), capi.ACT_F32, m, k,
                                              capi.ptr(y), capi.ACT_F32, n, capi.ptr(bg), capi.ptr(bu), capi.ACTFN_SILU,
                                              capi.MEM_HOST), dev.ctx)
        return y.reshape(lead + (n,))


    @staticmethod
    def forward_mlp(gate: "QMatMul", up: "QMatMul", down: "QMatMul", xs: np.ndarray) -> np.ndarray:
        """``(silu(x @ gate.T) * (x @ up.T)) @ down.T``, the whole of ``Qwen3MLP::forward`` (src/models/qwen3.rs:161-167),
        through ``turq_mlp``: the intermediate stays in f32 on the library's side."""
        xs = np.asarray(xs)
        k, n_out = gate.qtensor._k, down.qtensor._n
        if xs.ndim < 2 or xs.shape[-1] != k:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: input {xs.shape}, layers need last dim {k}")
        if xs.dtype != np.float32 or not xs.flags["C_CONTIGUOUS"]:
            raise TurqError(capi.ERR_INVALID, "forward_mlp needs a contiguous f32 input")
        lead = xs.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        y = np.empty((m, n_out), np.float32)
        dev = gate.qtensor.device
        capi.check(dev.L.turq_mlp(dev.ctx, gate.qtensor.handle, up.qtensor.handle, down.qtensor.handle, capi.ptr(xs), capi.ACT_F32, m, k,
                                  capi.ptr(y), capi.ACT_F32, n_out, None, None, None, capi.ACTFN_SILU, capi.MEM_HOST), dev.ctx)
        return y.reshape(lead + (n_out,))


class LinearX:
    """``LinearX::Quantized { qmatmul, bias }`` (src/models/layers/linear.rs:8-31)."""

    def __init__(self, qmatmul: QMatMul, bias: Optional[np.ndarray] = None):
        self.qmatmul = qmatmul
        self.bias = bias

    def forward(self, x: np.ndarray) -> np.ndarray:
        return self.qmatmul.forward(x, bias=self.bias)

    def forward_add(self, x: np.ndarray, residual: np.ndarray) -> np.ndarray:
        """``residual + forward(x)``: the residual connection of the decoder layer (``x + h``, src/models/qwen3.rs:635) taken
        into the matmul's store (``TURQ_OUT_ACCUMULATE``)."""
        q = self.qmatmul.qtensor
        n, k = q._n, q._k
        x = np.ascontiguousarray(x, np.float32)
        if x.ndim < 2 or x.shape[-1] != k:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: input {x.shape}, weight needs last dim {k}")
        lead = x.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        y = np.array(residual, np.float32, copy=True).reshape(-1)
        if y.size != m * n:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: the residual has {y.size} elements, the output {m * n}")
        b = None if self.bias is None else np.ascontiguousarray(self.bias, np.float32)
        dev = q.device
        algo = capi.ALGO_SIMPLE if self.qmatmul.dense else capi.ALGO_AUTO
        capi.check(dev.L.turq_qmatmul(dev.ctx, q.handle, capi.ptr(x), capi.ACT_F32, m, k, capi.ptr(y), capi.ACT_F32 | capi.OUT_ACCUMULATE,
                                      n, capi.ptr(b), capi.MEM_HOST, algo), dev.ctx)
        return y.reshape(lead + (n,))

    def __repr__(self) -> str:
        return "LinearX::Quantized"     # candle keeps dense GGUF tensors inside QMatMul too (QMatMul::Tensor)


class QVarBuilder:
    """``src/weights/gguf_varbuilder.rs``: GGUF header parsed once, tensors read lazily."""

    def __init__(self, device: Device, gguf, path: List[str], cache: list, layout: int):
        self._device = device
        self._g = gguf
        self._path = path
        self._cache = cache          # shared one-entry [name, tensor] cache
        self._layout = layout

    @classmethod
    def from_gguf(cls, p: str, device: Device, layout: int = capi.LAYOUT_TILED) -> "QVarBuilder":
        g = ctypes.c_void_p()
        capi.check(device.L.turq_gguf_open(str(p).encode(), ctypes.byref(g)))
        return cls(device, g, [], [None, None], layout)

    def pp(self, s) -> "QVarBuilder":
        return QVarBuilder(self._device, self._g, self._path + [str(s)], self._cache, self._layout)

    def path(self, tensor_name: str) -> str:
        return tensor_name if not self._path else ".".join(self._path) + "." + tensor_name

    def device(self) -> Device:
        return self._device

    def _load(self, full: str, shape) -> QTensor:
        L, dev = self._device.L, self._device
        dt, nd, nb = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
        dims = (ctypes.c_int64 * 4)()
        off = ctypes.c_uint64()
        capi.check(L.turq_gguf_tensor_info(self._g, full.encode(), ctypes.byref(dt), ctypes.byref(nd), dims, ctypes.byref(off),
                                           ctypes.byref(nb)))
        got = tuple(dims[i] for i in range(nd.value))
        layout = self._layout if dt.value in (capi.Q8_0, capi.Q4_K, capi.Q5_K, capi.Q6_K) else capi.LAYOUT_NATIVE
        h = ctypes.c_void_p()
        capi.check(L.turq_gguf_load_weight(dev.ctx, self._g, full.encode(), -1, -1, layout, ctypes.byref(h)), dev.ctx)
        t = QTensor(dev, h)
        t._one_dim = nd.value == 1
        return t

    def get(self, s, name: str) -> QTensor:
        shape = (s,) if isinstance(s, int) else tuple(s)
        full = self.path(name)
        if self._cache[0] == full:
            t = self._cache[1]
        else:
            t = self._load(full, shape)
            self._cache[0], self._cache[1] = full, t
        if t.shape() != shape:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch for {name}, got {list(t.shape())}, expected {list(shape)}")
        return t.clone()

    def get_no_shape(self, name: str) -> QTensor:
        return self._load(self.path(name), None)

    def contains_key(self, key: str) -> bool:
        return self._device.L.turq_gguf_tensor_info(self._g, self.path(key).encode(), None, None, None, None, None) == capi.OK

    def tensor_shape(self, key: str):
        nd = ctypes.c_int()
        dims = (ctypes.c_int64 * 4)()
        rc = self._device.L.turq_gguf_tensor_info(self._g, self.path(key).encode(), None, ctypes.byref(nd), dims, None, None)
        return None if rc != capi.OK else [dims[i] for i in range(nd.value)]

    def all_keys(self) -> List[str]:
        L = self._device.L
        return [L.turq_gguf_tensor_name(self._g, i).decode() for i in range(L.turq_gguf_tensor_count(self._g))]

    def metadata_u64(self, key: str) -> int:
        v = ctypes.c_uint64()
        capi.check(self._device.L.turq_gguf_meta_u64(self._g, key.encode(), ctypes.byref(v)))
        return v.value


def linear(in_dim: int, out_dim: int, vb: QVarBuilder) -> LinearX:
    """GGUF arm of ``layers::linear`` (src/models/layers/linear.rs:59-70): weight stays quantized, an optional
    bias tensor is dequantized at load."""
    qweight = vb.get((out_dim, in_dim), "weight")
    bias = None
    try:
        qbias = vb.get(out_dim, "bias")     # the reference looks the bias up with `.ok()`: absent or mis-shaped means none
    except TurqError:
        qbias = None
    if qbias is not None:
        bias = qbias.dequantize(vb.device()).reshape(-1)     # ... but a failing dequantize is an error (`.transpose()?`)
    return LinearX(QMatMul.from_arc(qweight), bias)


class NormX:
    """``NormX`` over candle_nn's ``RmsNorm`` (src/models/layers/norm.rs:9-41): the input is taken as it comes (f32 or f16 here),
    normalised in f32 and returned in the input's type."""

    def __init__(self, device: Device, weight: np.ndarray, eps: float):
        self.device = device
        self.weight = np.ascontiguousarray(weight, np.float32).reshape(-1)
        self.eps = float(eps)

    def forward(self, xs: np.ndarray) -> np.ndarray:
        xs = np.asarray(xs)
        k = self.weight.size
        if xs.ndim < 1 or xs.shape[-1] != k:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in rms-norm: last dim {xs.shape[-1] if xs.ndim else None} != {k}")
        if xs.dtype == np.float32:
            xt = capi.ACT_F32
        elif xs.dtype == np.float16:
            xt = capi.ACT_F16
        else:
            raise TurqError(capi.ERR_DTYPE, f"unsupported activation dtype {xs.dtype}")
        xs = np.ascontiguousarray(xs)
        m = xs.size // k if k else 0
        y = np.empty_like(xs)
        dev = self.device
        capi.check(dev.L.turq_rms_norm(dev.ctx, capi.ptr(xs), xt, m, k, k, capi.ptr(self.weight), self.eps, capi.ptr(y), xt, k,
                                       capi.MEM_HOST), dev.ctx)
        return y

    def forward_then(self, layers: "list[QMatMul]", xs: np.ndarray) -> "list[np.ndarray]":
        """``QMatMul.forward_multi(layers, self.forward(xs))`` in one call (``turq_norm_qmatmul_multi``): ln1 -> q / k / v
        (src/models/qwen3.rs:633-634, 272-274), the final norm -> lm_head."""
        import ctypes

        if not layers:
            return []
        xs = np.ascontiguousarray(xs, np.float32)
        k = self.weight.size
        if xs.ndim < 2 or xs.shape[-1] != k or any(l.qtensor._k != k for l in layers):
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch in matmul: input {xs.shape}, norm and layers need last dim {k}")
        if any(l.dense for l in layers):
            xn = self.forward(xs)
            return [l.forward(xn) for l in layers]
        lead = xs.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        cnt = len(layers)
        ys = [np.empty((m, l.qtensor._n), np.float32) for l in layers]
        warr = (ctypes.c_void_p * cnt)(*[l.qtensor.handle.value for l in layers])
        yarr = (ctypes.c_void_p * cnt)(*[y.ctypes.data for y in ys])
        ldys = (ctypes.c_int64 * cnt)(*[l.qtensor._n for l in layers])
        dev = self.device
        capi.check(dev.L.turq_norm_qmatmul_multi(dev.ctx, cnt, warr, capi.ptr(xs), capi.ACT_F32, m, k, capi.ptr(self.weight), self.eps, yarr,
                                                 capi.ACT_F32, ldys, None, capi.MEM_HOST), dev.ctx)
        return [y.reshape(lead + (y.shape[1],)) for y in ys]

    def forward_mlp_residual(self, gate: QMatMul, up: QMatMul, down: QMatMul, xs: np.ndarray) -> np.ndarray:
        """``xs + mlp(self.forward(xs))``, the second half of the decoder layer (src/models/qwen3.rs:637-640), in one call
        (``turq_norm_mlp`` with ``TURQ_OUT_ACCUMULATE``)."""
        xs = np.ascontiguousarray(xs, np.float32)
        k, n_out = gate.qtensor._k, down.qtensor._n
        if xs.ndim < 2 or xs.shape[-1] != k or n_out != k or self.weight.size != k:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch: input {xs.shape}, the MLP maps {k} features to {n_out}, the norm has {self.weight.size}")
        m = xs.size // k
        y = xs.copy()
        dev = self.device
        capi.check(dev.L.turq_norm_mlp(dev.ctx, gate.qtensor.handle, up.qtensor.handle, down.qtensor.handle, capi.ptr(xs), capi.ACT_F32, m, k,
                                       capi.ptr(self.weight), self.eps, capi.ptr(y), capi.ACT_F32 | capi.OUT_ACCUMULATE, n_out, None, None,
                                       None, capi.ACTFN_SILU, capi.MEM_HOST), dev.ctx)
        return y

    def __repr__(self) -> str:
        return "RmsNorm"


def rms_norm(size: int, eps: float, vb: QVarBuilder, is_gemma: bool = False) -> NormX:
    """GGUF arm of ``layers::norm::rms_norm`` (src/models/layers/norm.rs:52-94): the ``weight`` tensor dequantized to f32
    (plus one for the Gemma family)."""
    w = vb.get(size, "weight").dequantize(vb.device()).reshape(-1)
    if is_gemma:
        w = w + np.float32(1.0)
    return NormX(vb.device(), w, eps)


class Embedding:
    """candle's ``Embedding`` over a table that stays quantized in HBM: ``forward(ids)`` gathers and dequantizes the rows
    (``turq_embedding_lookup``) where the reference dequantizes the whole table at load (src/models/layers/mod.rs:30-37)."""

    def __init__(self, table: QTensor, hidden_size: int):
        if table._k != hidden_size:
            raise TurqError(capi.ERR_SHAPE, f"shape mismatch for weight, got [{table._n}, {table._k}], expected [*, {hidden_size}]")
        self.table = table
        self.hidden_size = hidden_size

    def forward(self, ids: np.ndarray) -> np.ndarray:
        ids = np.asarray(ids)
        if ids.dtype.kind not in "iu":
            raise TurqError(capi.ERR_DTYPE, f"token ids must be integers, got {ids.dtype}")
        if ids.size and (ids.min() < 0 or ids.max() >= self.table._n):
            raise TurqError(capi.ERR_INVALID, f"index outside the table of {self.table._n} rows")
        flat = np.ascontiguousarray(ids.reshape(-1), np.uint32)
        out = np.empty((flat.size, self.hidden_size), np.float32)
        dev = self.table.device
        capi.check(dev.L.turq_embedding_lookup(dev.ctx, self.table.handle, capi.ptr(flat), flat.size, capi.ptr(out), capi.ACT_F32,
                                               self.hidden_size, capi.MEM_HOST), dev.ctx)
        return out.reshape(ids.shape + (self.hidden_size,))


def embedding(vocab_size: Optional[int], hidden_size: int, vb: QVarBuilder) -> Tuple[Embedding, int]:
    """GGUF arm of ``layers::embedding`` (src/models/layers/mod.rs:11-50): the shape check when the vocabulary size is given,
    ``get_no_shape`` otherwise; returns the layer and the vocabulary size."""
    t = vb.get((vocab_size, hidden_size), "weight") if vocab_size is not None else vb.get_no_shape("weight")
    return Embedding(t, hidden_size), (vocab_size if vocab_size is not None else t._n)
