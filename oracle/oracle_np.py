"""NumPy restatement of the GGUF block formats (test infrastructure, NOT product code).

Second, independently written statement of what ``turq_oracle.c`` restates: candle-core
0.10.2 ``quantized/k_quants.rs`` (``to_float``, ``from_float``, ``vec_dot``) as reached from the
reference at ``src/models/layers/linear.rs:19-31`` (``QMatMul::forward``) and
``src/weights/mod.rs:150,161`` (``QTensor::dequantize``).  It is written per output ELEMENT
(gather by index arithmetic over whole arrays of blocks) where the C file walks pointers block by
block, so that an indexing slip in either one shows up as a bit difference between the two.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this.

PARITY UNPINNED for the same points as the C file: f32 operation order inside ``to_float`` and
the rounding rules of ``from_float`` cannot be checked against an executable candle here.
"""
from __future__ import annotations

import numpy as np

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, Q8_K, BF16 = 0, 1, 8, 12, 13, 14, 15, 30
BLOCK_ELEMS = {F32: 1, F16: 1, BF16: 1, Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256, Q8_K: 256}
BLOCK_BYTES = {F32: 4, F16: 2, BF16: 2, Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210, Q8_K: 292}

_f32 = np.float32


def _as_blocks(raw, dtype) -> np.ndarray:
    raw = np.ascontiguousarray(np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw)
    raw = raw.view(np.uint8).reshape(-1)
    bb = BLOCK_BYTES[dtype]
    if raw.size % bb:
        raise ValueError(f"{raw.size} bytes is not a whole number of {bb}-byte blocks")
    return raw.reshape(-1, bb)


def _f16_field(blk: np.ndarray, off: int) -> np.ndarray:
    """little-endian binary16 at byte offset ``off`` of every block, widened exactly to f32"""
    return np.ascontiguousarray(blk[:, off:off + 2]).view("<f2").reshape(-1).astype(_f32)


def scale_min_k4(scales: np.ndarray):
    """12 packed bytes -> (sc[8], m[8]) 6-bit values, stated as bit fields:
    sub-blocks 0..3: sc = low 6 bits of byte j,   m = low 6 bits of byte j+4;
    sub-blocks 4..7: sc = low nibble of byte j+4 with bits 6..7 of byte j-4 on top,
                     m  = high nibble of byte j+4 with bits 6..7 of byte j on top."""
    s = scales.astype(np.uint16)
    sc = np.empty(scales.shape[:-1] + (8,), np.uint8)
    mn = np.empty_like(sc)
    sc[..., 0:4] = s[..., 0:4] % 64
    mn[..., 0:4] = s[..., 4:8] % 64
    sc[..., 4:8] = (s[..., 8:12] % 16) + 16 * (s[..., 0:4] // 64)
    mn[..., 4:8] = (s[..., 8:12] // 16) + 16 * (s[..., 4:8] // 64)
    return sc, mn


def dequantize(dtype: int, raw) -> np.ndarray:
    """raw block bytes -> flat f32 array (bit-exact target of QTensor::dequantize)"""
    if dtype == F32:
        return np.frombuffer(bytes(raw), "<f4").astype(_f32)
    if dtype == F16:
        return np.frombuffer(bytes(raw), "<f2").astype(_f32)
    if dtype == BF16:
        u = np.frombuffer(bytes(raw), "<u2").astype(np.uint32) << 16
        return u.view(_f32)
    blk = _as_blocks(raw, dtype)
    nb = blk.shape[0]
    if dtype == Q8_0:
        d = _f16_field(blk, 0)
        q = blk[:, 2:34].view(np.int8).astype(_f32)
        return (q * d[:, None]).reshape(-1)
    e = np.arange(256)
    if dtype in (Q4_K, Q5_K):
        d = _f16_field(blk, 0)
        dmin = _f16_field(blk, 2)
        sc, mn = scale_min_k4(blk[:, 4:16])
        sub = e // 32                       # sub-block of element e
        byte = 32 * (e // 64) + (e % 32)    # qs byte that carries it
        hi = (e // 32) % 2                  # 0: low nibble, 1: high nibble
        qs = blk[:, 16:144] if dtype == Q4_K else blk[:, 48:176]
        nib = np.where(hi[None, :] == 1, qs[:, byte] >> 4, qs[:, byte] & 0xF).astype(_f32)
        if dtype == Q5_K:
            qh = blk[:, 16:48]
            bit = (qh[:, e % 32] >> sub[None, :].astype(np.uint8)) & 1     # bit `sub` of qh[e%32]
            nib = nib + np.where(bit == 1, _f32(16.0), _f32(0.0))
        dl = d[:, None] * sc[:, sub].astype(_f32)       # rounded to f32
        ml = dmin[:, None] * mn[:, sub].astype(_f32)    # rounded to f32
        prod = dl * nib                                  # rounded to f32
        return (prod - ml).astype(_f32).reshape(-1)
    if dtype == Q6_K:
        ql, qh, scb = blk[:, 0:128], blk[:, 128:192], blk[:, 192:208].view(np.int8)
        d = _f16_field(blk, 208)
        half = e // 128                 # which 128-element half
        r = e % 128
        quarter = r // 32               # 0..3 inside the half
        l = r % 32
        lbyte = 64 * half + l + 32 * (quarter % 2)
        lo = np.where((quarter // 2)[None, :] == 1, ql[:, lbyte] >> 4, ql[:, lbyte] & 0xF)
        h2 = (qh[:, 32 * half + l] >> (2 * quarter)[None, :].astype(np.uint8)) & 3
        q = (lo.astype(np.int16) + 16 * h2.astype(np.int16) - 32).astype(_f32)
        sc = scb[:, e // 16].astype(_f32)               # one int8 scale per 16 elements
        return ((d[:, None] * sc) * q).astype(_f32).reshape(-1)
    raise ValueError(f"unsupported dtype {dtype}")


def _round_half_away(v: np.ndarray) -> np.ndarray:
    """Rust f32::round on f32 input (exact: |v| < 2^23 has an exact .5 test in f32)"""
    v = v.astype(_f32)
    t = np.trunc(v)
    return np.where(np.abs(v - t) >= _f32(0.5), t + np.sign(v), t).astype(_f32)


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    """f32 [k] -> uint8 [k/32, 34]  (BlockQ8_0::from_float)"""
    x = np.asarray(x, _f32).reshape(-1, 32)
    amax = np.max(np.abs(x), axis=1)
    d = (amax / _f32(127.0)).astype(_f32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, _f32(1.0) / d, _f32(0.0)).astype(_f32)
    q = np.clip(_round_half_away(x * inv[:, None]), -128, 127).astype(np.int8)
    out = np.empty((x.shape[0], 34), np.uint8)
    out[:, 0:2] = d.astype("<f2").view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out


def quantize_q8_K(x: np.ndarray) -> np.ndarray:
    """f32 [k] -> uint8 [k/256, 292]  (BlockQ8K::from_float)"""
    x = np.asarray(x, _f32).reshape(-1, 256)
    nb = x.shape[0]
    ax = np.abs(x)
    first = np.argmax(ax, axis=1)                      # first index of the largest |x|
    mx = x[np.arange(nb), first]
    amax = ax[np.arange(nb), first]
    out = np.zeros((nb, 292), np.uint8)
    nz = amax != 0
    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = (_f32(-128.0) / mx).astype(_f32)
        v = _round_half_away((iscale[:, None] * x).astype(_f32))
        q = np.where(nz[:, None], np.clip(np.minimum(v, _f32(127.0)), -128, 127), 0).astype(np.int8)
        d = np.where(nz, (_f32(1.0) / iscale).astype(_f32), _f32(0.0)).astype(_f32)
    bs = q.reshape(nb, 16, 16).astype(np.int32).sum(axis=2).astype("<i2")
    out[:, 0:4] = d.astype("<f4").view(np.uint8).reshape(-1, 4)
    out[:, 4:260] = q.view(np.uint8)
    out[:, 260:292] = bs.view(np.uint8).reshape(nb, 32)
    return out


def int_weights(dtype: int, raw):
    """Integer view used by vec_dot: (a[nb,256|32] int, per-element integer scale, mins[nb,8] or None)."""
    blk = _as_blocks(raw, dtype)
    e = np.arange(256)
    if dtype == Q8_0:
        return blk[:, 2:34].view(np.int8).astype(np.int32), None, None
    if dtype in (Q4_K, Q5_K):
        sc, mn = scale_min_k4(blk[:, 4:16])
        qs = blk[:, 16:144] if dtype == Q4_K else blk[:, 48:176]
        byte = 32 * (e // 64) + (e % 32)
        a = np.where(((e // 32) % 2)[None, :] == 1, qs[:, byte] >> 4, qs[:, byte] & 0xF).astype(np.int32)
        if dtype == Q5_K:
            a = a + 16 * ((blk[:, 16:48][:, e % 32] >> (e // 32)[None, :].astype(np.uint8)) & 1).astype(np.int32)
        return a, sc[:, e // 32].astype(np.int32), mn.astype(np.int32)
    if dtype == Q6_K:
        ql, qh, scb = blk[:, 0:128], blk[:, 128:192], blk[:, 192:208].view(np.int8)
        half, r = e // 128, e % 128
        quarter, l = r // 32, r % 32
        lbyte = 64 * half + l + 32 * (quarter % 2)
        lo = np.where((quarter // 2)[None, :] == 1, ql[:, lbyte] >> 4, ql[:, lbyte] & 0xF).astype(np.int32)
        h2 = ((qh[:, 32 * half + l] >> (2 * quarter)[None, :].astype(np.uint8)) & 3).astype(np.int32)
        return lo + 16 * h2 - 32, scb[:, e // 16].astype(np.int32), None
    raise ValueError(dtype)


def qmatmul(dtype: int, x: np.ndarray, raw, n: int, k: int) -> np.ndarray:
    """candle CPU QMatMul::forward: quantise activations (Q8_K / Q8_0), integer dot per block,
    f32 scale.  The integer sums are exact; the final f32 accumulation runs block by block in
    the order of the scalar vec_dot (per block: 8 lane sums for the K-quants)."""
    x = np.asarray(x, _f32).reshape(-1, k)
    m = x.shape[0]
    out = np.empty((m, n), _f32)
    a, isc, mins = int_weights(dtype, raw)
    if dtype == Q8_0:
        nbr = k // 32
        wd = _f16_field(_as_blocks(raw, Q8_0), 0).reshape(n, nbr)
        a = a.reshape(n, nbr, 32)
        for r in range(m):
            xq = quantize_q8_0(x[r])
            yd = _f16_field(xq, 0)
            yq = xq[:, 2:].view(np.int8).astype(np.int32)
            sumi = np.einsum("nbj,bj->nb", a, yq).astype(_f32)
            acc = np.zeros(n, _f32)
            for b in range(nbr):
                acc = acc + (sumi[:, b] * wd[:, b]) * yd[b]
            out[r] = acc
        return out
    nbr = k // 256
    blk = _as_blocks(raw, dtype)
    if dtype == Q6_K:
        wd = _f16_field(blk, 208).reshape(n, nbr)
        wdmin = None
    else:
        wd = _f16_field(blk, 0).reshape(n, nbr)
        wdmin = _f16_field(blk, 2).reshape(n, nbr)
        mins = mins.reshape(n, nbr, 8)
    ws = (a * isc).reshape(n, nbr, 32, 8)          # scale folded in: integer, exact
    for r in range(m):
        xq = quantize_q8_K(x[r])
        yd = np.ascontiguousarray(xq[:, 0:4]).view("<f4").reshape(-1)
        yq = xq[:, 4:260].view(np.int8).astype(np.int32).reshape(nbr, 32, 8)
        bs = np.ascontiguousarray(xq[:, 260:292]).view("<i2").astype(np.int32).reshape(nbr, 8, 2).sum(axis=2)
        aux32 = np.einsum("nbgl,bgl->nbl", ws, yq)   # [n, nbr, 8] lane sums
        sums = np.zeros((n, 8), _f32)
        sumf = np.zeros(n, _f32)
        for b in range(nbr):
            dd = (wd[:, b] * yd[b]).astype(_f32)
            sums = sums + dd[:, None] * aux32[:, b, :].astype(_f32)
            if wdmin is not None:
                sumi = (mins[:, b, :] * bs[b][None, :]).sum(axis=1).astype(_f32)
                sumf = sumf - (wdmin[:, b] * yd[b]).astype(_f32) * sumi
        s = np.zeros(n, _f32)
        for l in range(8):
            s = s + sums[:, l]
        out[r] = sumf + s
    return out


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """``act(gate) * up`` of the reference's MLP, src/models/qwen3.rs:161-167 (``x.apply(&gate_proj)?.apply(&act_fn)? *
    x.apply(&up_proj)?``) with ``act_fn`` = SiLU, candle's ``v / (1 + exp(-v))``; evaluated in f64 and rounded once to f32.
    Pinned by closed forms (tests/test_oracle_kat.py): silu(0) = 0, silu(v) - silu(-v) = v, silu(v) -> v for large v,
    the minimum -0.27846 at v = -1.27846; candle's own f32 evaluation order is not reproduced (tolerance test, not bit test)."""
    g = np.asarray(gate, np.float64)
    with np.errstate(over="ignore"):
        act = g / (1.0 + np.exp(-g))
    return (act * np.asarray(up, np.float64)).astype(_f32)
