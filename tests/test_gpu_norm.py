"""turq_rms_norm against the formula in f64 (candle_nn's RmsNorm as the reference builds it in src/models/layers/norm.rs:52-94:
y = x / sqrt(mean(x^2) + eps) * weight, f32 arithmetic).  The f32 summation order of candle's kernel is not reproduced bit by bit
(parity unpinned at that level: candle-nn is not in the reference tree); the bar is 1e-6 relative, a few f32 ulps."""
import ctypes

import numpy as np
import pytest

from tests.helpers import Gpu, rel_l2
from tur_amd import capi, qlinear, synth
from tur_amd.gguf import write_gguf

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def want_norm(x, w, eps):
    x64 = np.asarray(x, np.float64)
    return x64 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + eps) * np.asarray(w, np.float64)


def call(gpu, x, w, eps, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32, mem=capi.MEM_HOST, ldx=None, ldy=None):
    m, k = x.shape
    ldx, ldy = ldx or k, ldy or k
    xb = np.zeros((m, ldx), np.float32)
    xb[:, :k] = x
    send = synth.to_bf16_bits(xb).reshape(m, ldx) if x_dtype == capi.ACT_BF16 else xb.astype(np.float16) if x_dtype == capi.ACT_F16 else xb
    ydt = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}[y_dtype]
    y = np.zeros((m, ldy), ydt)
    w = np.ascontiguousarray(w, np.float32)
    if mem == capi.MEM_DEVICE:
        xd, wd, yd = gpu.dev_buffer(send), gpu.dev_buffer(w), gpu.dev_buffer(y)
        capi.check(gpu.L.turq_rms_norm(gpu.ctx, xd, x_dtype, m, k, ldx, wd, eps, yd, y_dtype, ldy, mem), gpu.ctx)
        y = gpu.read_back(yd, (m, ldy), ydt)
        for p in (xd, wd, yd):
            gpu.dev_free(p)
    else:
        capi.check(gpu.L.turq_rms_norm(gpu.ctx, capi.ptr(send), x_dtype, m, k, ldx, capi.ptr(w), eps, capi.ptr(y), y_dtype, ldy, mem), gpu.ctx)
    if y_dtype == capi.ACT_BF16:
        y = synth.from_bf16_bits(y).reshape(m, ldy)
    return np.asarray(y, np.float32)[:, :k]


@pytest.mark.parametrize("mem", [capi.MEM_HOST, capi.MEM_DEVICE], ids=["host", "device"])
@pytest.mark.parametrize("m,k", [(1, 4096), (5, 1024), (64, 4096), (3, 5), (2, 4100), (7, 12288), (1, 1)])
def test_rms_norm_f32(gpu, m, k, mem):
    rng = np.random.default_rng(m * 1000 + k)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.01, 30, (m, 1))).astype(np.float32)
    w = rng.standard_normal(k).astype(np.float32)
    for eps in (1e-6, 1e-5):
        y = call(gpu, x, w, eps, mem=mem)
        assert rel_l2(y, want_norm(x, w, eps)) <= 1e-6


def test_rms_norm_types_strides_and_in_place(gpu):
    rng = np.random.default_rng(2)
    m, k = 6, 2048
    x = synth.random_activation(m, k, seed=3, bf16=True)
    w = rng.standard_normal(k).astype(np.float32)
    want = want_norm(x, w, 1e-6)
    assert rel_l2(call(gpu, x, w, 1e-6, x_dtype=capi.ACT_BF16), want) <= 1e-6                       # bf16 in, f32 out
    assert rel_l2(call(gpu, x, w, 1e-6, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16), want) <= 3e-3   # rounded once to bf16
    xh = x.astype(np.float16).astype(np.float32)
    assert rel_l2(call(gpu, xh, w, 1e-6, x_dtype=capi.ACT_F16, y_dtype=capi.ACT_F16), want_norm(xh, w, 1e-6)) <= 5e-4
    assert rel_l2(call(gpu, x, w, 1e-6, ldx=k + 24, ldy=k + 8, mem=capi.MEM_DEVICE), want) <= 1e-6    # row strides
    # in place on the device: y = x
    xd, wd = gpu.dev_buffer(x), gpu.dev_buffer(w)
    capi.check(gpu.L.turq_rms_norm(gpu.ctx, xd, capi.ACT_F32, m, k, k, wd, 1e-6, xd, capi.ACT_F32, k, capi.MEM_DEVICE), gpu.ctx)
    assert rel_l2(gpu.read_back(xd, (m, k), np.float32), want) <= 1e-6
    gpu.dev_free(xd)
    gpu.dev_free(wd)
    # rows of zeros stay zeros (eps keeps the root positive), huge rows stay finite
    z = np.zeros((2, k), np.float32)
    assert np.array_equal(call(gpu, z, w, 1e-6), z)
    big = (rng.standard_normal((2, k)) * 1e15).astype(np.float32)
    assert rel_l2(call(gpu, big, w, 1e-6), want_norm(big, w, 1e-6)) <= 1e-6


def test_rms_norm_errors(gpu):
    L, ctx = gpu.L, gpu.ctx
    x = np.zeros((2, 8), np.float32)
    w = np.ones(8, np.float32)
    y = np.zeros((2, 8), np.float32)
    args = lambda **kw: dict(dict(x=capi.ptr(x), xt=capi.ACT_F32, m=2, k=8, ldx=8, w=capi.ptr(w), eps=1e-6, y=capi.ptr(y), yt=capi.ACT_F32, ldy=8,
                                  mem=capi.MEM_HOST), **kw)
    def run(**kw):
        a = args(**kw)
        return L.turq_rms_norm(ctx, a["x"], a["xt"], a["m"], a["k"], a["ldx"], a["w"], a["eps"], a["y"], a["yt"], a["ldy"], a["mem"])
    assert run() == capi.OK
    assert run(ldx=7) == capi.ERR_SHAPE and run(ldy=7) == capi.ERR_SHAPE and run(m=-1) == capi.ERR_SHAPE
    assert run(xt=9) == capi.ERR_DTYPE and run(yt=9) == capi.ERR_DTYPE
    assert run(w=None) == capi.ERR_INVALID and run(mem=5) == capi.ERR_INVALID
    assert run(m=0) == capi.OK and run(k=0, ldx=0, ldy=0) == capi.OK
    assert L.turq_rms_norm(None, None, 0, 0, 0, 0, None, 0.0, None, 0, 0, 0) == capi.ERR_INVALID


def test_normx_from_a_gguf_file_feeds_the_projections(tmp_path):
    # the reference's order in a decoder layer: h = norm(x); q = q_proj(h)  (src/models/qwen3.rs)
    k, n = 512, 96
    rng = np.random.default_rng(9)
    nw = rng.standard_normal(k).astype("<f4")
    raw = synth.random_weight(capi.Q4_K, n, k, seed=4)
    path = tmp_path / "n.gguf"
    write_gguf(str(path), [("blk.0.attn_norm.weight", 0, (k,), nw.view(np.uint8)), ("blk.0.attn_q.weight", capi.Q4_K, (n, k), raw)])
    dev = qlinear.Device.new_hip(0)
    try:
        vb = qlinear.QVarBuilder.from_gguf(str(path), dev).pp("blk").pp(0)
        norm = qlinear.rms_norm(k, 1e-6, vb.pp("attn_norm"))
        gemma = qlinear.rms_norm(k, 1e-6, vb.pp("attn_norm"), is_gemma=True)
        q = qlinear.linear(k, n, vb.pp("attn_q"))
        assert repr(norm) == "RmsNorm" and np.array_equal(norm.weight, nw) and np.array_equal(gemma.weight, nw + np.float32(1))
        x = rng.standard_normal((2, 3, k)).astype(np.float32)
        h = norm.forward(x)
        assert h.shape == x.shape and rel_l2(h, want_norm(x, nw, 1e-6)) <= 1e-6
        from oracle import capi as orc
        y = q.forward(h)
        assert rel_l2(y, orc.matmul_dequant(capi.Q4_K, h.reshape(-1, k), raw, n, k).reshape(y.shape)) <= 1e-3
        with pytest.raises(capi.TurqError, match="shape mismatch"):
            norm.forward(np.zeros((2, k + 1), np.float32))
    finally:
        dev.close()
