"""RmsNorm taken into the forward calls: turq_norm_qmatmul_multi (q / k / v behind ln1, the LM head behind the final norm) and
turq_norm_mlp (x + mlp(ln2(x)) of the reference's decoder layer, src/models/qwen3.rs:633-640).

Checked against the f64 norm followed by the oracle's matmul on dequantized weights (1e-3), and against the separate calls
turq_rms_norm (f32 output) + turq_qmatmul_multi / turq_mlp: bit-equal wherever the call runs the norm into scratch or lets the
norm write the prefill GEMM's fragments, within 5e-4 where the one-row kernel applies the norm itself (it rounds x * weight to
f16 and scales the sums, where the separate calls round x / rms * weight: two roundings of about 2.4e-4 each against the exact row)."""
import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from oracle import oracle_np as onp
from tests.helpers import Gpu, rel_l2
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ACC = capi.OUT_ACCUMULATE
EPS = 1e-6


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def want_norm(x, w, eps=EPS):
    x64 = np.asarray(x, np.float64)
    return (x64 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + eps) * np.asarray(w, np.float64)).astype(np.float32)


def send(x, x_dtype):
    m, k = x.shape
    return synth.to_bf16_bits(x).reshape(m, k) if x_dtype == capi.ACT_BF16 else x.astype(np.float16) if x_dtype == capi.ACT_F16 else np.ascontiguousarray(x, np.float32)


class Dev:
    """device buffers of one test, freed together"""

    def __init__(self, gpu):
        self.gpu, self.ps = gpu, []

    def put(self, arr):
        p = self.gpu.dev_buffer(np.ascontiguousarray(arr))
        self.ps.append(p)
        return p

    def free(self):
        for p in self.ps:
            self.gpu.dev_free(p)


def norm_multi(gpu, ws, ns, x, nw, x_dtype=capi.ACT_F32, mem=capi.MEM_DEVICE, biases=None):
    L, ctx = gpu.L, gpu.ctx
    m, k = x.shape
    cnt = len(ws)
    outs = [np.zeros((m, n), np.float32) for n in ns]
    warr = (ctypes.c_void_p * cnt)(*[w.value for w in ws])
    ldys = (ctypes.c_int64 * cnt)(*ns)
    d = Dev(gpu)
    try:
        if mem == capi.MEM_DEVICE:
            xp, nwp = d.put(send(x, x_dtype)), d.put(np.asarray(nw, np.float32))
            yps = [d.put(o) for o in outs]
            bps = None if biases is None else [None if b is None else d.put(np.asarray(b, np.float32)) for b in biases]
        else:
            xs = send(x, x_dtype)
            nws = np.ascontiguousarray(nw, np.float32)
            xp, nwp = capi.ptr(xs), capi.ptr(nws)
            yps = [capi.ptr(o) for o in outs]
            bps = None if biases is None else [None if b is None else capi.ptr(np.ascontiguousarray(b, np.float32)) for b in biases]
        yarr = (ctypes.c_void_p * cnt)(*[p.value for p in yps])
        barr = None if bps is None else (ctypes.c_void_p * cnt)(*[None if p is None else p.value for p in bps])
        capi.check(L.turq_norm_qmatmul_multi(ctx, cnt, warr, xp, x_dtype, m, k, nwp, EPS, yarr, capi.ACT_F32, ldys, barr, mem), ctx)
        if mem == capi.MEM_DEVICE:
            outs = [gpu.read_back(p, (m, n), np.float32) for p, n in zip(yps, ns)]
    finally:
        d.free()
    return outs


def separate(gpu, ws, ns, x, nw, x_dtype=capi.ACT_F32, biases=None):
    """turq_rms_norm into an f32 buffer, then turq_qmatmul_multi on it (device pointers)"""
    L, ctx = gpu.L, gpu.ctx
    m, k = x.shape
    d = Dev(gpu)
    try:
        xp, nwp, xn = d.put(send(x, x_dtype)), d.put(np.asarray(nw, np.float32)), d.put(np.zeros((m, k), np.float32))
        capi.check(L.turq_rms_norm(ctx, xp, x_dtype, m, k, k, nwp, EPS, xn, capi.ACT_F32, k, capi.MEM_DEVICE), ctx)
        normed = gpu.read_back(xn, (m, k), np.float32)
    finally:
        d.free()
    return gpu.qmatmul_multi(ws, normed, ns, k, biases=biases), normed


QKV = [(Q4_K, 2048), (Q4_K, 512), (Q6_K, 512)]


@pytest.mark.parametrize("x_dtype", [capi.ACT_F32, capi.ACT_BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("m", [1, 2, 8, 32, 40, 200])
def test_norm_then_q_k_v(gpu, m, x_dtype):
    k = 2048
    raws = [synth.random_weight(dt, n, k, seed=10 + i) for i, (dt, n) in enumerate(QKV)]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for (dt, n), raw in zip(QKV, raws)]
    ns = [n for _, n in QKV]
    rng = np.random.default_rng(m)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.1, 20, (m, 1))).astype(np.float32)     # a residual stream: rows of any scale
    if x_dtype == capi.ACT_BF16:
        x = synth.from_bf16_bits(synth.to_bf16_bits(x)).reshape(m, k)
    nw = (1.0 + 0.3 * rng.standard_normal(k)).astype(np.float32)
    biases = [None, rng.standard_normal(ns[1]).astype(np.float32), None]
    got = norm_multi(gpu, ws, ns, x, nw, x_dtype=x_dtype, biases=biases)
    sep, _ = separate(gpu, ws, ns, x, nw, x_dtype=x_dtype, biases=biases)
    xn = want_norm(x, nw)
    for (dt, n), raw, y, s, b in zip(QKV, raws, got, sep, biases):
        want = orc.matmul_dequant(dt, xn, raw, n, k) + (0 if b is None else b)
        assert rel_l2(y, want) <= 1e-3, (dt, n, rel_l2(y, want))
        if m == 1:
            assert rel_l2(y, s) <= 5e-4, (dt, n, rel_l2(y, s))      # both round the normalised row to f16, at different points
        else:
            assert np.array_equal(y, s), (dt, n, m)
    for w in ws:
        gpu.release(w)


@pytest.mark.parametrize("fmts", [[(Q6_K, 512)], [(Q4_K, 768), (Q6_K, 256)], [(13, 512), (Q6_K, 256)]], ids=["q6k", "q4k+q6k", "q5k+q6k"])
def test_one_row_on_a_wide_hidden_size(gpu, fmts):
    # 12288 columns are 48 column tiles: 3 per wave, where the plain one-row kernels keep three in flight; with the norm weights
    # next to them the kernels of the fused call keep two (three spill registers) - same sums, same bars
    k, m = 12288, 1
    raws = [synth.random_weight(dt, n, k, seed=20 + i) for i, (dt, n) in enumerate(fmts)]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for (dt, n), raw in zip(fmts, raws)]
    ns = [n for _, n in fmts]
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((m, k)) * 3).astype(np.float32)
    nw = (1.0 + 0.3 * rng.standard_normal(k)).astype(np.float32)
    got = norm_multi(gpu, ws, ns, x, nw)
    sep, _ = separate(gpu, ws, ns, x, nw)
    xn = want_norm(x, nw)
    for (dt, n), raw, y, s in zip(fmts, raws, got, sep):
        assert rel_l2(y, orc.matmul_dequant(dt, xn, raw, n, k)) <= 1e-3, (dt, n)
        assert rel_l2(y, s) <= 5e-4, (dt, n, rel_l2(y, s))
    for w in ws:
        gpu.release(w)


def test_final_norm_then_lm_head_and_host_pointers(gpu):
    n, k = 5000, 1024
    raw = synth.random_weight(Q6_K, n, k, seed=3)
    w = gpu.upload(Q6_K, n, k, raw, capi.LAYOUT_TILED)
    rng = np.random.default_rng(0)
    nw = (1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    for m in (1, 3):
        x = (rng.standard_normal((m, k)) * 7).astype(np.float32)
        want = orc.matmul_dequant(Q6_K, want_norm(x, nw), raw, n, k)
        assert rel_l2(norm_multi(gpu, [w], [n], x, nw)[0], want) <= 1e-3
        assert rel_l2(norm_multi(gpu, [w], [n], x, nw, mem=capi.MEM_HOST)[0], want) <= 1e-3
    # rows of zeros stay zeros (the norm divides by sqrt(eps)), and nothing is left uncounted
    z = norm_multi(gpu, [w], [n], np.zeros((1, k), np.float32), nw)[0]
    assert np.all(z == 0)
    gpu.release(w)


@pytest.mark.parametrize("m", [1, 4, 32, 48, 160])
def test_norm_mlp_adds_to_the_residual_stream(gpu, m):
    n_ff, k = 3072, 1024
    raws = [synth.random_weight(Q4_K, n_ff, k, seed=1), synth.random_weight(Q4_K, n_ff, k, seed=2), synth.random_weight(Q6_K, k, n_ff, seed=3)]
    ws = [gpu.upload(Q4_K, n_ff, k, raws[0], capi.LAYOUT_TILED), gpu.upload(Q4_K, n_ff, k, raws[1], capi.LAYOUT_TILED),
          gpu.upload(Q6_K, k, n_ff, raws[2], capi.LAYOUT_TILED)]
    L, ctx = gpu.L, gpu.ctx
    rng = np.random.default_rng(m)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.5, 4, (m, 1))).astype(np.float32)
    nw = (0.02 * (1.0 + 0.3 * rng.standard_normal(k))).astype(np.float32)       # small: keeps the synthetic intermediate inside f16
    d = Dev(gpu)
    try:
        xp, nwp = d.put(x), d.put(nw)
        yp = d.put(x.copy())                                                   # the residual stream: y = x + mlp(norm(x))
        capi.check(L.turq_norm_mlp(ctx, ws[0], ws[1], ws[2], xp, capi.ACT_F32, m, k, nwp, EPS, yp, capi.ACT_F32 | ACC, k, None, None, None,
                                   0, capi.MEM_DEVICE), ctx)
        got = gpu.read_back(yp, (m, k), np.float32)
        # the separate calls: norm (f32), turq_mlp, the sum on the host
        xn = d.put(np.zeros((m, k), np.float32))
        capi.check(L.turq_rms_norm(ctx, xp, capi.ACT_F32, m, k, k, nwp, EPS, xn, capi.ACT_F32, k, capi.MEM_DEVICE), ctx)
        normed = gpu.read_back(xn, (m, k), np.float32)
    finally:
        d.free()
    sep = gpu.mlp(*ws, normed, n_ff, k, k) + x
    xn64 = want_norm(x, nw)
    h = onp.silu_mul(orc.matmul_dequant(Q4_K, xn64, raws[0], n_ff, k), orc.matmul_dequant(Q4_K, xn64, raws[1], n_ff, k))
    want = orc.matmul_dequant(Q6_K, h, raws[2], k, n_ff) + x
    assert rel_l2(got - x, want - x) <= (1e-3 if m <= 32 else 2e-3), rel_l2(got - x, want - x)
    if m == 1:
        assert rel_l2(got - x, sep - x) <= 1.5e-3      # (two different f16 roundings of the row, carried through SiLU and down_proj)
    else:
        assert np.array_equal(got, sep), m
    for w in ws:
        gpu.release(w)


def test_errors_are_reported(gpu):
    L, ctx = gpu.L, gpu.ctx
    raw = synth.random_weight(Q4_K, 64, 256, seed=1)
    w = gpu.upload(Q4_K, 64, 256, raw, capi.LAYOUT_TILED)
    x = np.zeros((1, 256), np.float32)
    nw = np.ones(256, np.float32)
    y = np.zeros((1, 64), np.float32)
    warr = (ctypes.c_void_p * 1)(w.value)
    yarr = (ctypes.c_void_p * 1)(y.ctypes.data)
    ldys = (ctypes.c_int64 * 1)(64)
    call = lambda xp=capi.ptr(x), nwp=capi.ptr(nw), ldx=256, xt=capi.ACT_F32: L.turq_norm_qmatmul_multi(
        ctx, 1, warr, xp, xt, 1, ldx, nwp, EPS, yarr, capi.ACT_F32, ldys, None, capi.MEM_HOST)
    assert call() == capi.OK
    assert call(nwp=None) == capi.ERR_INVALID
    assert call(xp=None) == capi.ERR_INVALID
    assert call(ldx=100) == capi.ERR_SHAPE
    assert call(xt=7) == capi.ERR_DTYPE
    assert L.turq_norm_mlp(ctx, w, w, None, capi.ptr(x), capi.ACT_F32, 1, 256, capi.ptr(nw), EPS, capi.ptr(y), capi.ACT_F32, 64, None, None, None,
                           0, capi.MEM_HOST) == capi.ERR_INVALID
    gpu.release(w)
