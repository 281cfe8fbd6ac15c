"""GPU parity of turq_qmatmul_gate_up: act(x gate^T) * (x up^T), the first half of the reference's MLP
(src/models/qwen3.rs:161-167, src/models/granite_41.rs:151-155), called through the C ABI.

Checked against the oracle's matmul on dequantized weights (f16-rounded activations where the MFMA kernels run, which is
every case here) followed by the oracle's SiLU product; bar 1e-3 relative L2 like the matmul itself, and a sharper 5e-5 that
an indexing slip (gate and up exchanged, a row of the pair taken twice) cannot pass.
"""
import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from oracle import oracle_np as onp
from tests.helpers import Gpu, rel_l2
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ALL = [Q8_0, Q4_K, Q5_K, Q6_K]


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def f16_round(x):
    return x.astype(np.float16).astype(np.float32)


def expected(dt, x, raw_g, raw_u, n, k, bg=None, bu=None):
    g = orc.matmul_dequant(dt, x, raw_g, n, k)
    u = orc.matmul_dequant(dt, x, raw_u, n, k)
    if bg is not None:
        g = g + bg
    if bu is not None:
        u = u + bu
    return onp.silu_mul(g, u)


@pytest.mark.parametrize("dt", ALL)
@pytest.mark.parametrize("m", [1, 2, 3, 8, 16, 20, 32, 40])
def test_gate_up_matches_the_two_calls(gpu, dt, m):
    # one row: inside the one-row kernel; up to 32 rows: inside the prepared-fragment kernel; m = 40: the two GEMM products + the
    # elementwise pass
    n, k = 200, 1024 + (64 if dt == Q8_0 else 0)
    raw_g = synth.random_weight(dt, n, k, seed=dt + 1)
    raw_u = synth.random_weight(dt, n, k, seed=dt + 2)
    wg = gpu.upload(dt, n, k, raw_g, capi.LAYOUT_TILED)
    wu = gpu.upload(dt, n, k, raw_u, capi.LAYOUT_TILED)
    x = synth.random_activation(m, k, seed=m)
    y = gpu.gate_up(wg, wu, x, n, k)
    want = expected(dt, f16_round(x), raw_g, raw_u, n, k)
    assert y.shape == (m, n)
    assert rel_l2(y, want) <= (5e-5 if m <= 32 else 1e-3), rel_l2(y, want)
    assert rel_l2(y, expected(dt, x, raw_g, raw_u, n, k)) <= 1e-3
    # the same numbers as the two separate calls combined on the host
    g = gpu.qmatmul(wg, x, n, k)
    u = gpu.qmatmul(wu, x, n, k)
    assert rel_l2(y, onp.silu_mul(g, u)) <= 2e-5
    # exchanged weights give something else (the expression is not symmetric)
    assert rel_l2(gpu.gate_up(wu, wg, x, n, k), want) > 0.1
    gpu.release(wg)
    gpu.release(wu)


@pytest.mark.parametrize("dt", [Q4_K, Q6_K])
def test_gate_up_two_rows_on_large_weights(gpu, dt):
    # 2 x 5 MiB and more: two activation rows stay in the one-row kernel (Q4_K: one packed pair)
    n, k = 4100, 4096
    raw_g = synth.random_weight(dt, n, k, seed=11)
    raw_u = synth.random_weight(dt, n, k, seed=12)
    wg = gpu.upload(dt, n, k, raw_g, capi.LAYOUT_TILED)
    wu = gpu.upload(dt, n, k, raw_u, capi.LAYOUT_TILED)
    for m in (1, 2):
        x = synth.random_activation(m, k, seed=20 + m)
        bg = np.random.default_rng(1).standard_normal(n).astype(np.float32)
        bu = np.random.default_rng(2).standard_normal(n).astype(np.float32)
        y = gpu.gate_up(wg, wu, x, n, k, bias_gate=bg, bias_up=bu, ldx=k + 8, ldy=n + 3)
        assert rel_l2(y, expected(dt, f16_round(x), raw_g, raw_u, n, k, bg, bu)) <= 5e-5, m
        xb = synth.random_activation(m, k, seed=30 + m, bf16=True)
        yb = gpu.gate_up(wg, wu, xb, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16)
        assert rel_l2(yb, expected(dt, xb, raw_g, raw_u, n, k)) <= 4e-3, m      # bf16 store
        # (f16 activations; an f16 OUTPUT could not hold these synthetic products, which pass 65504)
        yh = gpu.gate_up(wg, wu, f16_round(x), n, k, x_dtype=capi.ACT_F16)
        assert rel_l2(yh, expected(dt, f16_round(x), raw_g, raw_u, n, k)) <= 5e-5, m
    gpu.release(wg)
    gpu.release(wu)


@pytest.mark.parametrize("dt", ALL)
def test_gate_up_several_rows_bias_strides_and_stores(gpu, dt):
    # the prepared-fragment form on a pair large enough for several waves per workgroup: biases, row strides, bf16 in and out
    n, k = 1030, 4096 + (32 if dt == Q8_0 else 0)
    raw_g = synth.random_weight(dt, n, k, seed=61)
    raw_u = synth.random_weight(dt, n, k, seed=62)
    wg = gpu.upload(dt, n, k, raw_g, capi.LAYOUT_TILED)
    wu = gpu.upload(dt, n, k, raw_u, capi.LAYOUT_TILED)
    bg = np.random.default_rng(3).standard_normal(n).astype(np.float32)
    bu = np.random.default_rng(4).standard_normal(n).astype(np.float32)
    for m in (5, 16, 29):
        x = synth.random_activation(m, k, seed=70 + m, bf16=True)
        want = expected(dt, x, raw_g, raw_u, n, k, bg, bu)
        y = gpu.gate_up(wg, wu, x, n, k, bias_gate=bg, bias_up=bu, ldx=k + 8, ldy=n + 2)
        assert rel_l2(y, want) <= 5e-5, m
        yb = gpu.gate_up(wg, wu, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16, bias_gate=bg, bias_up=bu)
        assert rel_l2(yb, want) <= 4e-3, m
    gpu.release(wg)
    gpu.release(wu)


def test_gate_up_wide_k_and_host_memory(gpu):
    # 48 column tiles (the down-projection's width); host pointers take the two host-path products
    n, k = 512, 12288
    raw_g = synth.random_weight(Q4_K, n, k, seed=41)
    raw_u = synth.random_weight(Q4_K, n, k, seed=42)
    wg = gpu.upload(Q4_K, n, k, raw_g, capi.LAYOUT_TILED)
    wu = gpu.upload(Q4_K, n, k, raw_u, capi.LAYOUT_TILED)
    x = synth.random_activation(1, k, seed=43)
    want = expected(Q4_K, f16_round(x), raw_g, raw_u, n, k)
    assert rel_l2(gpu.gate_up(wg, wu, x, n, k), want) <= 5e-5
    yh = gpu.gate_up(wg, wu, x, n, k, mem=capi.MEM_HOST, y_dtype=capi.ACT_BF16)
    assert rel_l2(yh, want) <= 4e-3
    assert rel_l2(gpu.gate_up(wg, wu, x, n, k, mem=capi.MEM_HOST), want) <= 5e-5
    xs = x * np.float32(1 / 64)      # products small enough for an f16 store
    ws = expected(Q4_K, f16_round(xs), raw_g, raw_u, n, k)
    assert np.abs(ws).max() < 60000
    assert rel_l2(gpu.gate_up(wg, wu, xs, n, k, y_dtype=capi.ACT_F16), ws) <= 5e-4
    assert rel_l2(gpu.gate_up(wg, wu, xs, n, k, y_dtype=capi.ACT_F16, mem=capi.MEM_HOST), ws) <= 5e-4
    gpu.release(wg)
    gpu.release(wu)


def test_gate_up_native_layout_and_mixed_formats(gpu):
    # nothing the fused kernel takes: native layout, or gate and up of different formats
    n, k = 96, 512
    raws = {dt: synth.random_weight(dt, n, k, seed=dt) for dt in (Q4_K, Q6_K)}
    x = synth.random_activation(2, k, seed=5)
    wg = gpu.upload(Q4_K, n, k, raws[Q4_K], capi.LAYOUT_NATIVE)
    wu = gpu.upload(Q4_K, n, k, raws[Q4_K], capi.LAYOUT_NATIVE)
    g = orc.matmul_dequant(Q4_K, x, raws[Q4_K], n, k)
    assert rel_l2(gpu.gate_up(wg, wu, x, n, k), onp.silu_mul(g, g)) <= 5e-5
    gpu.release(wg)
    gpu.release(wu)
    wg = gpu.upload(Q4_K, n, k, raws[Q4_K], capi.LAYOUT_TILED)
    wu = gpu.upload(Q6_K, n, k, raws[Q6_K], capi.LAYOUT_TILED)
    xr = f16_round(x)
    want = onp.silu_mul(orc.matmul_dequant(Q4_K, xr, raws[Q4_K], n, k), orc.matmul_dequant(Q6_K, xr, raws[Q6_K], n, k))
    assert rel_l2(gpu.gate_up(wg, wu, x, n, k), want) <= 5e-5
    gpu.release(wg)
    gpu.release(wu)


def test_gate_up_errors_and_empty(gpu):
    L, ctx = gpu.L, gpu.ctx
    n, k = 32, 256
    raw = synth.random_weight(Q4_K, n, k, seed=1)
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_TILED)
    w2 = gpu.upload(Q4_K, n + 16, k, synth.random_weight(Q4_K, n + 16, k, seed=2), capi.LAYOUT_TILED)
    x = np.zeros((1, k), np.float32)
    y = np.full((1, n), 7.0, np.float32)
    args = (capi.ptr(x), capi.ACT_F32, 1, k, capi.ptr(y), capi.ACT_F32, n, None, None)
    assert L.turq_qmatmul_gate_up(ctx, w, w2, *args, 0, capi.MEM_HOST) == capi.ERR_SHAPE
    assert "gate is" in capi.last_error(ctx)
    assert L.turq_qmatmul_gate_up(ctx, w, w, *args, 5, capi.MEM_HOST) == capi.ERR_INVALID          # unknown activation
    assert L.turq_qmatmul_gate_up(ctx, w, None, *args, 0, capi.MEM_HOST) == capi.ERR_INVALID
    assert L.turq_qmatmul_gate_up(ctx, w, w, capi.ptr(x), capi.ACT_F32, 1, k, capi.ptr(y), capi.ACT_F32, n - 1, None, None, 0,
                                  capi.MEM_HOST) == capi.ERR_SHAPE                                    # ldy < n
    assert L.turq_qmatmul_gate_up(ctx, w, w, capi.ptr(x), capi.ACT_F32, -1, k, capi.ptr(y), capi.ACT_F32, n, None, None, 0,
                                  capi.MEM_HOST) == capi.ERR_SHAPE
    assert np.all(y == 7.0)
    # m = 0 is a no-op; zero activations give silu(0) * 0 = 0
    assert L.turq_qmatmul_gate_up(ctx, w, w, capi.ptr(x), capi.ACT_F32, 0, k, capi.ptr(y), capi.ACT_F32, n, None, None, 0,
                                  capi.MEM_HOST) == capi.OK
    assert np.all(y == 7.0)
    assert np.all(gpu.gate_up(w, w, x, n, k) == 0.0)
    gpu.release(w)
    gpu.release(w2)


def test_gate_up_in_a_graph(gpu):
    # decode step: fused gate / up, then down, captured once and replayed with other activations
    L, ctx = gpu.L, gpu.ctx
    hid, ffn = 1024, 3072
    raws = [synth.random_weight(Q4_K, ffn, hid, seed=1), synth.random_weight(Q4_K, ffn, hid, seed=2),
            synth.random_weight(Q6_K, hid, ffn, seed=3)]
    wg = gpu.upload(Q4_K, ffn, hid, raws[0], capi.LAYOUT_TILED)
    wu = gpu.upload(Q4_K, ffn, hid, raws[1], capi.LAYOUT_TILED)
    wd = gpu.upload(Q6_K, hid, ffn, raws[2], capi.LAYOUT_TILED)

    def dev(nbytes):
        p = ctypes.c_void_p()
        capi.check(L.turq_dev_alloc(ctx, nbytes, ctypes.byref(p)), ctx)
        return p
    xd, hd, yd = dev(hid * 4), dev(ffn * 4), dev(hid * 4)
    capi.check(L.turq_graph_begin(ctx), ctx)
    capi.check(L.turq_qmatmul_gate_up(ctx, wg, wu, xd, capi.ACT_F32, 1, hid, hd, capi.ACT_F32, ffn, None, None, 0, capi.MEM_DEVICE), ctx)
    capi.check(L.turq_qmatmul(ctx, wd, hd, capi.ACT_F32, 1, ffn, yd, capi.ACT_F32, hid, None, capi.MEM_DEVICE, capi.ALGO_AUTO), ctx)
    graph = ctypes.c_void_p()
    capi.check(L.turq_graph_end(ctx, ctypes.byref(graph)), ctx)
    for seed in (1, 2, 3):
        # (scaled down: the synthetic weights are large, and the intermediate feeds f16 arithmetic in down_proj)
        x = synth.random_activation(1, hid, seed=seed) * np.float32(1 / 64)
        capi.check(L.turq_memcpy_h2d(ctx, xd, capi.ptr(x), x.nbytes), ctx)
        capi.check(L.turq_graph_launch(ctx, graph), ctx)
        capi.check(L.turq_sync(ctx), ctx)
        y = np.zeros((1, hid), np.float32)
        capi.check(L.turq_memcpy_d2h(ctx, capi.ptr(y), yd, y.nbytes), ctx)
        h = expected(Q4_K, f16_round(x), raws[0], raws[1], ffn, hid)
        assert np.abs(h).max() < 60000
        want = orc.matmul_dequant(Q6_K, f16_round(h), raws[2], hid, ffn)
        assert rel_l2(y, want) <= 1e-3, seed      # the f16 rounding of the intermediate sits on both sides, at slightly different values
    L.turq_graph_destroy(graph)
    for p in (xd, hd, yd):
        capi.check(L.turq_dev_free(ctx, p), ctx)
    for w in (wg, wu, wd):
        gpu.release(w)
