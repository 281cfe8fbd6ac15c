"""Seeded synthetic GGUF blocks and activations for tests and benchmarks.

Weights follow the ggml block layouts byte for byte, so what these functions return is what
``gguf_file::Content::tensor`` would hand to ``QTensor`` for a tensor of shape ``(n, k)``
(reference: ``src/weights/gguf_varbuilder.rs:72-74``).  Value distributions:

* Q8_0: int8 quants uniform in [-127, 127], scale ``d = f16(|N(0,1)| * 0.02)``;
* Q4_K / Q5_K: ``d, dmin = f16(|N(0,1)| * 0.01)``, eight 6-bit scales and mins uniform in 0..63
  packed into 12 bytes, quant bytes (and the Q5_K high-bit plane) uniform;
* Q6_K: ``ql`` / ``qh`` bytes uniform, sixteen int8 scales uniform in [-64, 63],
  ``d = f16(|N(0,1)| * 0.01)``;
* activations ~ N(0, 1) in f32 (optionally rounded to bf16).
"""
from __future__ import annotations

import numpy as np

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 8, 12, 13, 14, 30
BLOCK_ELEMS = {F32: 1, F16: 1, BF16: 1, Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256}
BLOCK_BYTES = {F32: 4, F16: 2, BF16: 2, Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210}
DTYPE_NAMES = {F32: "F32", F16: "F16", BF16: "BF16", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K"}
NAME_TO_DTYPE = {v: k for k, v in DTYPE_NAMES.items()}


def weight_nbytes(dtype: int, n: int, k: int) -> int:
    be = BLOCK_ELEMS[dtype]
    if k % be:
        raise ValueError(f"k={k} is not a multiple of the {DTYPE_NAMES[dtype]} block size {be}")
    return n * (k // be) * BLOCK_BYTES[dtype]


def pack_scales_mins(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """[..., 8] six-bit scales and mins -> [..., 12] packed bytes (inverse of the K-quant unpack)."""
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    q = np.empty(sc.shape[:-1] + (12,), np.uint8)
    q[..., 0:4] = sc[..., 0:4] | ((sc[..., 4:8] >> 4) << 6)
    q[..., 4:8] = mn[..., 0:4] | ((mn[..., 4:8] >> 4) << 6)
    q[..., 8:12] = (sc[..., 4:8] & 0xF) | ((mn[..., 4:8] & 0xF) << 4)
    return q


def _f16_bytes(v: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(v.astype("<f2")).view(np.uint8).reshape(-1, 2)


def random_blocks(dtype: int, nblocks: int, rng: np.random.Generator) -> np.ndarray:
    """uint8 [nblocks, block_bytes] of seeded random blocks."""
    bb = BLOCK_BYTES[dtype]
    out = np.empty((nblocks, bb), np.uint8)
    if dtype == Q8_0:
        out[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(nblocks, np.float32)) * np.float32(0.02))
        out[:, 2:] = rng.integers(-127, 128, (nblocks, 32), np.int8).view(np.uint8)
    elif dtype in (Q4_K, Q5_K):
        out[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(nblocks, np.float32)) * np.float32(0.01))
        out[:, 2:4] = _f16_bytes(np.abs(rng.standard_normal(nblocks, np.float32)) * np.float32(0.01))
        sc = rng.integers(0, 64, (nblocks, 8), np.uint8)
        mn = rng.integers(0, 64, (nblocks, 8), np.uint8)
        out[:, 4:16] = pack_scales_mins(sc, mn)
        out[:, 16:] = rng.integers(0, 256, (nblocks, bb - 16), np.uint8)
    elif dtype == Q6_K:
        out[:, 0:192] = rng.integers(0, 256, (nblocks, 192), np.uint8)
        out[:, 192:208] = rng.integers(-64, 64, (nblocks, 16), np.int8).view(np.uint8)
        out[:, 208:210] = _f16_bytes(np.abs(rng.standard_normal(nblocks, np.float32)) * np.float32(0.01))
    else:
        raise ValueError(f"no random block generator for dtype {dtype}")
    return out


def random_weight(dtype: int, n: int, k: int, seed: int) -> np.ndarray:
    """Flat uint8 array holding a [n, k] weight: n rows of k/blk consecutive blocks."""
    be = BLOCK_ELEMS[dtype]
    if k % be:
        raise ValueError(f"k={k} is not a multiple of the block size {be}")
    rng = np.random.default_rng(seed)
    return random_blocks(dtype, n * (k // be), rng).reshape(-1)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def random_activation(m: int, k: int, seed: int, bf16: bool = False) -> np.ndarray:
    """f32 [m, k] ~ N(0,1); with ``bf16`` the values are rounded to bf16 (still returned as f32)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k), np.float32)
    if bf16:
        x = from_bf16_bits(to_bf16_bits(x)).reshape(m, k)
    return x


# The shapes the headline metric is quoted on (Qwen3-8B, Qwen3-0.6B gate_proj).
QWEN3_8B = {
    "hidden": 4096, "ffn": 12288, "q_out": 4096, "kv_out": 1024, "vocab": 151936, "layers": 36,
}
CONFIGS = {
    "q8_0_gate_0p6b": [("gate", Q8_0, 3072, 1024)],
    "q4k_mlp_8b": [("gate", Q4_K, 12288, 4096), ("up", Q4_K, 12288, 4096), ("down", Q4_K, 4096, 12288)],
    "q4km_layer_8b": [
        ("q", Q4_K, 4096, 4096), ("k", Q4_K, 1024, 4096), ("v", Q6_K, 1024, 4096), ("o", Q4_K, 4096, 4096),
        ("gate", Q4_K, 12288, 4096), ("up", Q4_K, 12288, 4096), ("down", Q6_K, 4096, 12288),
    ],
    "q4k_prefill_up_8b": [("up", Q4_K, 12288, 4096)],
    "lm_head_q6k_8b": [("output", Q6_K, 151936, 4096)],
    "lm_head_q5k_8b": [("output", Q5_K, 151936, 4096)],
}
