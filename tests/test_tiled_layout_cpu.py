"""CPU checks of the tiled HBM layout (no GPU needed).

1. tile -> untile is the identity on GGUF bytes for every format, ragged row counts included.
2. A NumPy model of what one wave of the MFMA kernel does with a tile (same masks, same magic
   constants, same fused multiply-adds, same lane <-> (row, group) mapping as
   tur_amd/csrc/gemv_mfma.hip) reproduces x @ dequantize(W).T of the oracle.  This pins the bit
   positions documented in tur_amd/csrc/layout.h against the kernel's unpack arithmetic before
   anything runs on a GPU.
"""
import numpy as np
import pytest

from oracle import capi as orc
from tur_amd import capi, synth

Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
TILE_BYTES = {Q4_K: 2304, Q5_K: 2816, Q6_K: 3360, Q8_0: 4352}


def tile(dt, n, k, raw):
    L = capi.lib()
    out = np.zeros(L.turq_tiled_nbytes(dt, n, k), np.uint8)
    capi.check(L.turq_tile_host(dt, n, k, capi.ptr(raw), capi.ptr(out)))
    return out


@pytest.mark.parametrize("dt", [Q8_0, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("n,k", [(1, 256), (16, 512), (37, 1024), (130, 768)])
def test_tile_untile_roundtrip(dt, n, k):
    L = capi.lib()
    raw = synth.random_weight(dt, n, k, seed=n * 1000 + k + dt)
    t = tile(dt, n, k, raw)
    assert t.size == ((n + 15) // 16) * ((k + 255) // 256) * TILE_BYTES[dt]
    back = np.full_like(raw, 0xAA)
    capi.check(L.turq_untile_host(dt, n, k, capi.ptr(t), capi.ptr(back)))
    assert np.array_equal(raw, back)


def test_q8_0_ragged_columns_roundtrip():
    # k = 96: three blocks in a 256-column tile, the other five stay zero blocks
    L = capi.lib()
    raw = synth.random_weight(Q8_0, 20, 96, seed=3)
    t = tile(Q8_0, 20, 96, raw)
    back = np.zeros_like(raw)
    capi.check(L.turq_untile_host(Q8_0, 20, 96, capi.ptr(t), capi.ptr(back)))
    assert np.array_equal(raw, back)


def test_tile_rejects_bad_shapes():
    L = capi.lib()
    buf = np.zeros(4096, np.uint8)
    assert L.turq_tile_host(Q4_K, 4, 100, capi.ptr(buf), capi.ptr(buf)) == capi.ERR_SHAPE
    assert L.turq_tile_host(0, 4, 256, capi.ptr(buf), capi.ptr(buf)) == capi.ERR_SHAPE
    assert L.turq_tiled_nbytes(Q4_K, 4, 100) == 0


# ---------------------------------------------------------------------------------------------
# NumPy model of the kernel's per-lane arithmetic
# ---------------------------------------------------------------------------------------------
f16 = np.float16


def h2(u32):
    """packed dword(s) -> (lo, hi) f16 values"""
    u32 = np.asarray(u32, np.uint32)
    lo = (u32 & 0xFFFF).astype(np.uint16).view(f16)
    hi = (u32 >> 16).astype(np.uint16).view(f16)
    return lo, hi


def pk_fma(u32, s, c):
    """v_pk_fma_f16 on both halves: exact product + addend, one rounding to f16"""
    lo, hi = h2(u32)
    f = lambda v: (v.astype(np.float64) * np.float64(s) + np.float64(c)).astype(f16)
    return f(lo), f(hi)


def rotr(v, s):
    v = np.asarray(v, np.uint32)
    s = int(s) & 31
    return v if s == 0 else ((v >> np.uint32(s)) | (v << np.uint32(32 - s))).astype(np.uint32)


def lanes():
    L = np.arange(64)
    return L, L & 15, L >> 4


def k45_b_operands(tile_bytes, dt):
    """-> B[step 0..7][lane][slot 0..7] (f16, exact integers), bmin[lane][8], d[lane], dmin[lane]"""
    L, r, g = lanes()
    w32 = tile_bytes.view(np.uint32)
    qa = w32[0:256].reshape(64, 4)
    qb = w32[256:512].reshape(64, 4)
    hdr_off = 2048 if dt == Q4_K else 2560
    hd = tile_bytes[hdr_off:hdr_off + 256].view(np.uint32).reshape(16, 4)[r]          # [64, 4]
    if dt == Q5_K:
        hh = tile_bytes[2048:2560].view(np.uint32).reshape(64, 2)
    field = hd[:, 1].astype(object) | (hd[:, 2].astype(object) << 32) | (hd[:, 3].astype(object) << 64)
    G = np.array([(int(f) >> (24 * int(gg))) & 0xFFFFFF for f, gg in zip(field, g)], np.uint32)
    sc_lo, m_lo, sc_hi, m_hi = G & 63, (G >> 6) & 63, (G >> 12) & 63, (G >> 18) & 63
    d = (hd[:, 0] & 0xFFFF).astype(np.uint16).view(f16).astype(np.float32)
    dmin = (hd[:, 0] >> 16).astype(np.uint16).view(f16).astype(np.float32)
    B = np.zeros((8, 64, 8), f16)
    for i in range(8):
        w = (qa[:, i] if i < 4 else qb[:, i - 4]).astype(np.uint32)
        s = (sc_lo if i < 4 else sc_hi).astype(np.float64)
        w8 = w >> np.uint32(8)
        t = [(w & 0x000F000F) | 0x64006400, (w & 0x00F000F0) | 0x64006400,
             (w8 & 0x000F000F) | 0x64006400, (w8 & 0x00F000F0) | 0x64006400]
        if dt == Q5_K:
            u0 = 2 * i
            t[0] = t[0] | (rotr(hh[:, 0], u0) & 0x00100010)
            t[1] = t[1] | (rotr(hh[:, 1], u0) & 0x01000100)
            t[2] = t[2] | (rotr(hh[:, 0], u0 + 1) & 0x00100010)
            t[3] = t[3] | (rotr(hh[:, 1], u0 + 1) & 0x01000100)
        for tt in range(4):
            scale, addend = (s, -1024.0 * s) if tt % 2 == 0 else (s / 16.0, -64.0 * s)
            lo, hi = h2(t[tt])
            B[i, :, 2 * tt] = (lo.astype(np.float64) * scale + addend).astype(f16)
            B[i, :, 2 * tt + 1] = (hi.astype(np.float64) * scale + addend).astype(f16)
    bmin = np.zeros((64, 8), f16)
    bmin[:, 0:4] = m_lo[:, None]
    bmin[:, 4:8] = m_hi[:, None]
    return B, bmin, d, dmin


def q6_b_operands(tile_bytes):
    L, r, g = lanes()
    w32 = tile_bytes[:3072].view(np.uint32)
    qla, qlb, qh = w32[0:256].reshape(64, 4), w32[256:512].reshape(64, 4), w32[512:768].reshape(64, 4)
    sc = tile_bytes[3072:3328].view(np.int8).reshape(64, 4).astype(np.float64)
    d = tile_bytes[3328:3360].view(f16)[r].astype(np.float32)
    B1 = np.zeros((8, 64, 8), f16)
    B2 = np.zeros((8, 64, 8), f16)
    for i in range(8):
        s = sc[:, i // 2]
        w = (qla[:, i] if i < 4 else qlb[:, i - 4]).astype(np.uint32)
        w8 = rotr(w, 8)
        parts = [((w & 0x003C003C) | 0x5C005C00, s, -256 * s), ((w & 0x03C003C0) | 0x4C004C00, s, -16 * s),
                 ((w8 & 0x003C003C) | 0x5C005C00, s, -256 * s), ((w8 & 0x03C003C0) | 0x4C004C00, s, -16 * s)]
        hA = qh[:, i // 2] if i % 2 == 0 else rotr(qh[:, i // 2], 8)
        hB = rotr(hA, 4)
        hparts = [((hA & 0x00C000C0) | 0x4C004C00, 16 * s, -288 * s), ((hA & 0x03000300) | 0x44004400, 16 * s, -96 * s),
                  ((hB & 0x00C000C0) | 0x4C004C00, 16 * s, -288 * s), ((hB & 0x03000300) | 0x44004400, 16 * s, -96 * s)]
        for tt in range(4):
            for dst, (u, sca, add) in ((B1, parts[tt]), (B2, hparts[tt])):
                lo, hi = h2(u)
                dst[i, :, 2 * tt] = (lo.astype(np.float64) * sca + add).astype(f16)
                dst[i, :, 2 * tt + 1] = (hi.astype(np.float64) * sca + add).astype(f16)
    return B1, B2, d


def q8_b_operands(tile_bytes):
    L, r, g = lanes()
    planes = tile_bytes[:4096].view(np.uint32).reshape(4, 64, 4)
    dd = tile_bytes[4096:4352].view(f16).reshape(16, 8)[r].astype(np.float32)      # [64, 8]
    B = np.zeros((8, 64, 8), f16)
    for q in range(8):
        w0 = planes[q >> 1][:, (q & 1) * 2]
        w1 = planes[q >> 1][:, (q & 1) * 2 + 1]
        regs = [(w0 & 0x00FF00FF) | 0x64006400, ((w0 >> np.uint32(8)) & 0x00FF00FF) | 0x64006400,
                (w1 & 0x00FF00FF) | 0x64006400, ((w1 >> np.uint32(8)) & 0x00FF00FF) | 0x64006400]
        for tt in range(4):
            lo, hi = h2(regs[tt])
            B[q, :, 2 * tt] = (lo.astype(np.float32) - np.float32(1152)).astype(f16)
            B[q, :, 2 * tt + 1] = (hi.astype(np.float32) - np.float32(1152)).astype(f16)
    return B, dd


def mfma(A, B):
    """A[m][g][slot], B[lane = n + 16 g][slot] -> D[m][n] (f64 accumulate stands in for the f32 MFMA)"""
    Bn = B.reshape(4, 16, 8).astype(np.float64)          # [g][n][slot]
    return np.einsum("mgj,gnj->mn", A.astype(np.float64), Bn)


def model_gemv(dt, n, k, raw, x):
    """y[m, n] through the tiled layout and the kernel's arithmetic; x is rounded to f16 first."""
    m = x.shape[0]
    t = tile(dt, n, k, raw)
    ntc = (k + 255) // 256
    xh = np.zeros((m, ntc * 256), f16)
    xh[:, :k] = x.astype(f16)
    y = np.zeros((m, ((n + 15) // 16) * 16), np.float64)
    tb = TILE_BYTES[dt]
    for rt in range((n + 15) // 16):
        for b in range(ntc):
            tl = t[(rt * ntc + b) * tb:(rt * ntc + b + 1) * tb]
            xb = xh[:, 256 * b:256 * b + 256]
            if dt == Q8_0:
                B, dd = q8_b_operands(tl)
                for q in range(8):
                    A = xb[:, 32 * q:32 * q + 32].reshape(m, 4, 8)                 # [m][g][slot]
                    y[:, 16 * rt:16 * rt + 16] += mfma(A, B[q]) * dd[:16, q][None, :]
                continue
            A = xb.reshape(m, 4, 8, 8)                                              # [m][g][step][slot]
            if dt == Q6_K:
                B1, B2, d = q6_b_operands(tl)
                tmp = sum(mfma(A[:, :, i, :], B1[i]) + mfma(A[:, :, i, :], B2[i]) for i in range(8))
                y[:, 16 * rt:16 * rt + 16] += tmp * d[:16][None, :]
            else:
                B, bmin, d, dmin = k45_b_operands(tl, dt)
                tmp = sum(mfma(A[:, :, i, :], B[i]) for i in range(8))
                gs = xb.astype(np.float32).reshape(m, 4, 4, 16).sum(axis=3)         # 16-element group sums
                hi = gs.astype(f16)
                lo = (gs - hi.astype(np.float32)).astype(f16)
                S = np.stack([hi, lo], axis=-1).reshape(m, 4, 8)                     # (hi0, lo0, hi1, lo1, ...)
                tmin = mfma(S, bmin)
                y[:, 16 * rt:16 * rt + 16] += tmp * d[:16][None, :] - tmin * dmin[:16][None, :]
    return y[:, :n]


@pytest.mark.parametrize("dt", [Q4_K, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("n,k,m", [(16, 256, 1), (40, 768, 3)])
def test_kernel_model_matches_oracle(dt, n, k, m):
    raw = synth.random_weight(dt, n, k, seed=17 * dt + n)
    x = synth.random_activation(m, k, seed=99 + dt)
    xh = x.astype(f16).astype(np.float32)          # the kernel sees f16-rounded activations
    want = orc.matmul_dequant(dt, xh, raw, n, k)
    got = model_gemv(dt, n, k, raw, x)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel < 2e-6, rel


def test_kernel_model_weights_are_exact_integers():
    """Every B operand value is an integer below 2048 in magnitude (exact in f16) — Q6_K's high
    part may reach 4096 but only as a multiple of 16."""
    for dt in (Q4_K, Q5_K):
        raw = synth.random_weight(dt, 16, 256, seed=dt)
        B, _, _, _ = k45_b_operands(tile(dt, 16, 256, raw), dt)
        v = B.astype(np.float64)
        assert np.all(v == np.round(v)) and np.abs(v).max() <= (945 if dt == Q4_K else 1953)
    raw = synth.random_weight(Q6_K, 16, 256, seed=6)
    raw.reshape(-1, 210)[:, 192:208] = np.random.default_rng(0).integers(-128, 128, (16, 16), np.int8).view(np.uint8)
    B1, B2, _ = q6_b_operands(tile(Q6_K, 16, 256, raw))
    assert np.abs(B1.astype(np.float64)).max() <= 1920
    v2 = B2.astype(np.float64)
    assert np.all(v2 % 16 == 0) and np.abs(v2).max() <= 4096
