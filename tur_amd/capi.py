"""ctypes binding of ``libturq.so`` — one Python function per ``include/turq.h`` entry point."""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libturq.so")

OK, ERR_INVALID, ERR_SHAPE, ERR_DTYPE, ERR_HIP, ERR_OOM, ERR_IO, ERR_NOT_FOUND = range(8)
F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 8, 12, 13, 14, 30
ACT_F32, ACT_BF16, ACT_F16 = 0, 1, 2
OUT_ACCUMULATE = 0x100
LAYOUT_NATIVE, LAYOUT_TILED = 0, 1
MEM_HOST, MEM_DEVICE = 0, 1
ALGO_AUTO, ALGO_SIMPLE, ALGO_GEMV, ALGO_GEMM = 0, 1, 2, 3
ACTFN_SILU = 0
NOALLOC_SCRATCH_BYTES = 16 << 20

# every symbol include/turq.h declares: (restype, argtypes)
_SIGS = {
    "turq_version": (c_char_p, []),
    "turq_block_elems": (c_int, [c_int]),
    "turq_block_bytes": (c_int, [c_int]),
    "turq_weight_nbytes": (c_size_t, [c_int, c_int64, c_int64]),
    "turq_ctx_create": (c_int, [c_int, POINTER(c_void_p)]),
    "turq_ctx_destroy": (None, [c_void_p]),
    "turq_last_error": (c_char_p, [c_void_p]),
    "turq_sync": (c_int, [c_void_p]),
    "turq_ctx_stream": (c_void_p, [c_void_p]),
    "turq_ctx_set_wide_activations": (c_int, [c_void_p, c_int]),
    "turq_ctx_nonfinite_count": (c_int, [c_void_p, POINTER(c_uint64), c_int]),
    "turq_ctx_device_info": (c_int, [c_void_p, c_char_p, c_size_t, POINTER(c_int)]),
    "turq_dev_alloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "turq_dev_free": (c_int, [c_void_p, c_void_p]),
    "turq_memcpy_h2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "turq_memcpy_d2h": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "turq_weight_upload": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_size_t, c_int, POINTER(c_void_p)]),
    "turq_weight_retain": (c_int, [c_void_p]),
    "turq_weight_release": (c_int, [c_void_p]),
    "turq_weight_info": (c_int, [c_void_p, POINTER(c_int), POINTER(c_int64), POINTER(c_int64), POINTER(c_int), POINTER(c_size_t)]),
    "turq_weight_export": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "turq_tiled_nbytes": (c_size_t, [c_int, c_int64, c_int64]),
    "turq_tile_host": (c_int, [c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "turq_untile_host": (c_int, [c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "turq_dequantize": (c_int, [c_void_p, c_void_p, c_void_p, c_int]),
    "turq_embedding_lookup": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int]),
    "turq_rms_norm": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_float, c_void_p, c_int, c_int64, c_int]),
    "turq_qmatmul": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p, c_int, c_int]),
    "turq_qmatmul_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p]),
    "turq_qmatmul_multi": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p, c_void_p,
                                   c_int, c_int]),
    "turq_qmatmul_gate_up": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64,
                                     c_void_p, c_void_p, c_int, c_int]),
    "turq_mlp": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64,
                         c_void_p, c_void_p, c_void_p, c_int, c_int]),
    "turq_norm_qmatmul_multi": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_float, c_void_p, c_int,
                                        c_void_p, c_void_p, c_int]),
    "turq_norm_mlp": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_float, c_void_p, c_int,
                              c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int]),
    "turq_weight_prefetch": (c_int, [c_void_p, c_void_p]),
    "turq_quantize_q8_0": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int]),
    "turq_quantize_q8_k": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int]),
    "turq_read_yardstick": (c_int, [c_void_p, c_void_p, c_size_t]),
    "turq_prefill_plan": (c_int, [c_int, c_int64, c_int64, c_int64, c_int, POINTER(c_int), POINTER(c_int), POINTER(c_int)]),
    "turq_prefill_plan_multi": (c_int, [c_int, c_int64, c_int64, c_int64, c_int, c_int, POINTER(c_int)]),
    "turq_tuning_describe": (c_int, [c_char_p, c_size_t, POINTER(c_size_t)]),
    "turq_graph_begin": (c_int, [c_void_p]),
    "turq_graph_end": (c_int, [c_void_p, POINTER(c_void_p)]),
    "turq_graph_launch": (c_int, [c_void_p, c_void_p]),
    "turq_graph_destroy": (None, [c_void_p]),
    "turq_ctx_scratch_info": (c_int, [c_void_p, POINTER(c_int), POINTER(c_int), POINTER(c_size_t)]),
    "turq_profile_begin": (c_int, [c_void_p]),
    "turq_profile_end": (c_int, [c_void_p, POINTER(c_int64), POINTER(c_double)]),
    "turq_gguf_open": (c_int, [c_char_p, POINTER(c_void_p)]),
    "turq_gguf_close": (None, [c_void_p]),
    "turq_gguf_last_error": (c_char_p, [c_void_p]),
    "turq_gguf_tensor_count": (c_int64, [c_void_p]),
    "turq_gguf_tensor_name": (c_char_p, [c_void_p, c_int64]),
    "turq_gguf_tensor_info": (c_int, [c_void_p, c_char_p, POINTER(c_int), POINTER(c_int), POINTER(c_int64), POINTER(c_uint64), POINTER(c_size_t)]),
    "turq_gguf_meta_u64": (c_int, [c_void_p, c_char_p, POINTER(c_uint64)]),
    "turq_gguf_meta_f64": (c_int, [c_void_p, c_char_p, POINTER(c_double)]),
    "turq_gguf_meta_str": (c_int, [c_void_p, c_char_p, c_char_p, c_size_t]),
    "turq_gguf_read_tensor": (c_int, [c_void_p, c_char_p, c_void_p, c_size_t]),
    "turq_gguf_load_weight": (c_int, [c_void_p, c_void_p, c_char_p, c_int64, c_int64, c_int, POINTER(c_void_p)]),
}

_lib = None


class TurqError(RuntimeError):
    """A libturq call returned a non-zero status (the reference's candle_core::Error)."""

    def __init__(self, code: int, message: str):
        super().__init__(f"turq error {code}: {message}")
        self.code = code
        self.message = message


def lib() -> ctypes.CDLL:
    """Load libturq.so (built in-tree by ``__graft_entry__.build()`` / ``make -C tur_amd/csrc``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `make -C tur_amd/csrc` (there is no CPU fallback)")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def declared_symbols():
    return sorted(_SIGS)


def last_error(ctx=None) -> str:
    msg = lib().turq_last_error(ctx)
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc: int, ctx=None):
    if rc != OK:
        raise TurqError(rc, last_error(ctx))


def ptr(a) -> c_void_p:
    """host pointer of a numpy array, or pass an int / None through"""
    if a is None:
        return c_void_p(None)
    if isinstance(a, np.ndarray):
        return a.ctypes.data_as(c_void_p)
    return c_void_p(int(a))
