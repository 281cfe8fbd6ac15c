"""f32 activations of any finite magnitude (the reference's contract, src/weights/mod.rs:84-99: candle's CPU path scales every
256-element block of the activations on its own): calls on host pointers and, after turq_ctx_set_wide_activations, calls on
device pointers stay within the 1e-3 bar for rows far outside the f16 range; non-finite inputs propagate."""
import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu, rel_l2
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
MAGNITUDES = [1e-12, 1e-6, 1.0, 1e5, 1e20]


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def rows_of_mixed_magnitude(m, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    scale = np.array([MAGNITUDES[i % len(MAGNITUDES)] for i in range(m)], np.float32)[:, None]
    return (x * scale).astype(np.float32)


def per_row_rel(y, want):
    y, want = np.asarray(y, np.float64), np.asarray(want, np.float64)
    return np.linalg.norm(y - want, axis=1) / np.maximum(np.linalg.norm(want, axis=1), 1e-300)


@pytest.mark.parametrize("dt", [Q8_0, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("m", [1, 2, 5, 20, 40, 100])          # one-row kernel, batch kernels, prefill GEMM
def test_host_calls_take_any_f32_magnitude(gpu, dt, m):
    n, k = 208, 1024
    raw = synth.random_weight(dt, n, k, seed=dt + m)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    x = rows_of_mixed_magnitude(m, k, seed=m)
    bias = np.random.default_rng(1).standard_normal(n).astype(np.float32) * 1e-3
    y = gpu.qmatmul(w, x, n, k, bias=bias, mem=capi.MEM_HOST)
    want = orc.matmul_dequant(dt, x, raw, n, k).astype(np.float64) + bias
    assert np.all(np.isfinite(y))
    assert per_row_rel(y, want).max() <= 1e-3          # every row on its own: a tiny row must not drown next to a huge one
    gpu.release(w)


@pytest.mark.parametrize("x_dtype", [capi.ACT_F32, capi.ACT_BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("y_dtype", [capi.ACT_F32, capi.ACT_BF16], ids=["to-f32", "to-bf16"])
def test_device_calls_after_the_switch(x_dtype, y_dtype):
    g = Gpu()
    try:
        L, ctx = g.L, g.ctx
        dt, n, k = Q4_K, 320, 2048
        raw = synth.random_weight(dt, n, k, seed=3)
        w = g.upload(dt, n, k, raw, capi.LAYOUT_TILED)
        for m in (1, 8, 64):
            x = rows_of_mixed_magnitude(m, k, seed=10 + m)
            if x_dtype == capi.ACT_BF16:
                x = synth.from_bf16_bits(synth.to_bf16_bits(x)).reshape(m, k)
            want = orc.matmul_dequant(dt, x, raw, n, k)
            # without the switch rows of 1e5 and more overflow f16: infinities or NaNs, not a crash
            y = g.qmatmul(w, x, n, k, x_dtype=x_dtype, y_dtype=y_dtype)
            big = np.abs(x).max(axis=1) >= 65504
            assert m == 1 or (big.any() and not np.all(np.isfinite(y[big])))
            capi.check(L.turq_ctx_set_wide_activations(ctx, 1), ctx)
            y = g.qmatmul(w, x, n, k, x_dtype=x_dtype, y_dtype=y_dtype)
            assert np.all(np.isfinite(y))
            assert per_row_rel(y, want).max() <= (1e-3 if y_dtype == capi.ACT_F32 else 4e-3)
            capi.check(L.turq_ctx_set_wide_activations(ctx, 0), ctx)
        g.release(w)
    finally:
        g.close()


def test_more_rows_than_a_grid_has_rows_of_workgroups():
    # 70 000 rows on device pointers under the switch: the kernel that takes the row factors out again walks the rows in a
    # loop (a grid's second dimension ends at 65 535), so the rows past that are results too, not what the buffer held before
    g = Gpu()
    try:
        L, ctx = g.L, g.ctx
        dt, n, k, m = Q4_K, 128, 1024, 70000
        raw = synth.random_weight(dt, n, k, seed=6)
        w = g.upload(dt, n, k, raw, capi.LAYOUT_TILED)
        x = np.random.default_rng(8).standard_normal((m, k)).astype(np.float32)
        rows = np.array([0, 1, 65534, 65535, 65536, 65537, 69998, 69999])
        x[rows[::2]] *= 1e6
        capi.check(L.turq_ctx_set_wide_activations(ctx, 1), ctx)
        y = g.qmatmul(w, x, n, k, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32)
        assert np.all(np.isfinite(y))
        assert per_row_rel(y[rows], orc.matmul_dequant(dt, x[rows], raw, n, k)).max() <= 1e-3
        # every 1000th row as well, and no row left at zero
        some = np.arange(0, m, 1000)
        assert per_row_rel(y[some], orc.matmul_dequant(dt, x[some], raw, n, k)).max() <= 1e-3
        assert np.all(np.abs(y).max(axis=1) > 0)
        g.release(w)
    finally:
        g.close()


def test_grouped_calls_and_gate_up_under_the_switch():
    from oracle import oracle_np as onp
    g = Gpu()
    try:
        capi.check(g.L.turq_ctx_set_wide_activations(g.ctx, 1), g.ctx)
        k, ns, dts = 1024, [96, 48, 160], (Q4_K, Q4_K, Q6_K)
        raws = [synth.random_weight(dt, n, k, seed=n) for dt, n in zip(dts, ns)]
        ws = [g.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
        for m in (1, 6, 48):
            x = rows_of_mixed_magnitude(m, k, seed=m)
            for y, dt, n, raw in zip(g.qmatmul_multi(ws, x, ns, k), dts, ns, raws):
                assert per_row_rel(y, orc.matmul_dequant(dt, x, raw, n, k)).max() <= 1e-3
        # gate / up: SiLU is not homogeneous, so the rows go back to their own scale before it is applied
        n = 128
        rg, ru = synth.random_weight(Q4_K, n, k, seed=5), synth.random_weight(Q4_K, n, k, seed=6)
        wg, wu = g.upload(Q4_K, n, k, rg, capi.LAYOUT_TILED), g.upload(Q4_K, n, k, ru, capi.LAYOUT_TILED)
        x = rows_of_mixed_magnitude(5, k, seed=2)
        x[np.abs(x).max(axis=1) > 1e10] *= 1e-12        # keep gate * up inside f32
        y = g.gate_up(wg, wu, x, n, k)
        want = onp.silu_mul(orc.matmul_dequant(Q4_K, x, rg, n, k), orc.matmul_dequant(Q4_K, x, ru, n, k))
        assert per_row_rel(y, want).max() <= 2e-3
    finally:
        g.close()


def test_non_finite_activations_propagate(gpu):
    dt, n, k = Q4_K, 64, 512
    raw = synth.random_weight(dt, n, k, seed=8)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    x = np.random.default_rng(0).standard_normal((4, k)).astype(np.float32)
    x[1, 7] = np.inf
    x[2, 300] = np.nan
    y = gpu.qmatmul(w, x, n, k, mem=capi.MEM_HOST)
    want = orc.matmul_dequant(dt, x[[0, 3]], raw, n, k)
    assert rel_l2(y[[0, 3]], want) <= 1e-3                      # the finite rows are untouched
    assert not np.any(np.isfinite(y[1])) and np.all(np.isnan(y[2]))
    gpu.release(w)


def nonfinite(g, reset=1):
    n = ctypes.c_uint64(12345)
    capi.check(g.L.turq_ctx_nonfinite_count(g.ctx, ctypes.byref(n), reset), g.ctx)
    return n.value


@pytest.mark.parametrize("m", [1, 8, 48])
def test_a_finite_f32_result_that_no_bf16_holds_is_counted(m):
    # Q8_0 rows of all 127 with block scale 1: y = 127 * sum(x).  The rows are chosen so that y = 3.399e38: a finite f32, but
    # past the midpoint between the largest bf16 (3.3895e38) and 2^128, so the bf16 store rounds it to an infinity.  With wide
    # activations on (the rows are far outside f16) the f32 output is finite and nothing is counted; the bf16 output is counted.
    g = Gpu()
    try:
        L, ctx = g.L, g.ctx
        n, k = 32, 256
        block = np.concatenate([np.array([1.0], np.float16).view(np.uint8), np.full(32, 127, np.int8).view(np.uint8)])
        raw = np.tile(block, n * (k // 32))
        w = g.upload(Q8_0, n, k, raw, capi.LAYOUT_TILED)
        x = np.full((m, k), 3.399e38 / (127.0 * k), np.float32)
        capi.check(L.turq_ctx_set_wide_activations(ctx, 1), ctx)
        nonfinite(g)
        y32 = g.qmatmul(w, x, n, k, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_F32)
        assert np.all(np.isfinite(y32)) and np.all(np.abs(y32 / 3.399e38 - 1) < 1e-3)
        assert nonfinite(g) == 0
        y16 = g.qmatmul(w, x, n, k, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_BF16)
        assert np.all(np.isinf(y16))
        assert nonfinite(g) >= 1
        # a little lower and the bf16 store is the largest finite bf16: not counted
        y16 = g.qmatmul(w, x * np.float32(0.99), n, k, x_dtype=capi.ACT_F32, y_dtype=capi.ACT_BF16)
        assert np.all(np.isfinite(y16)) and nonfinite(g) == 0
        g.release(w)
    finally:
        g.close()


@pytest.mark.parametrize("m", [1, 2, 8, 24, 40, 100])     # one-row kernel, two rows, staged rows, prepared fragments, prefill GEMM
@pytest.mark.parametrize("dt", [Q4_K, Q6_K, Q8_0])
def test_overflow_on_device_pointers_is_counted(dt, m):
    """Wide activations off, device pointers, a finite row of magnitude 1e5: the call returns TURQ_OK and every kernel exits
    normally, the row comes out as infinities / NaNs, and turq_ctx_nonfinite_count sees it; rows inside the f16 range leave the
    count at zero, and so does the same input with wide activations on."""
    g = Gpu()
    try:
        L, ctx = g.L, g.ctx
        n, k = 208, 1024
        raw = synth.random_weight(dt, n, k, seed=dt + m)
        w = g.upload(dt, n, k, raw, capi.LAYOUT_TILED)
        nonfinite(g)                                   # whatever earlier tests of this process left behind
        x = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
        y = g.qmatmul_device(w, x, n, k)
        assert np.all(np.isfinite(y)) and nonfinite(g, reset=0) == 0
        x[m // 2] *= np.float32(1e5)
        y = g.qmatmul_device(w, x, n, k)
        assert not np.all(np.isfinite(y[m // 2]))
        assert nonfinite(g, reset=0) > 0
        assert nonfinite(g, reset=1) > 0 and nonfinite(g) == 0          # sticky until it is reset
        capi.check(L.turq_ctx_set_wide_activations(ctx, 1), ctx)
        y = g.qmatmul_device(w, x, n, k)
        assert np.all(np.isfinite(y)) and per_row_rel(y, orc.matmul_dequant(dt, x, raw, n, k)).max() <= 1e-3
        assert nonfinite(g) == 0
        g.release(w)
    finally:
        g.close()


@pytest.mark.parametrize("m", [1, 8, 32, 48, 160])
def test_mlp_intermediate_outside_f16_is_counted_and_wide_handles_it(m):
    """turq_mlp keeps act(gate) * up as f16 where down_proj's kernels would round it to f16 anyway: an intermediate of magnitude
    65520 and more is an infinity there.  With wide activations off the call still returns TURQ_OK and the count says so; with
    wide activations on the intermediate stays f32, its rows are scaled for down_proj, and the result is finite and within the
    bar of the oracle's chain."""
    from oracle import oracle_np as onp
    g = Gpu()
    try:
        L, ctx = g.L, g.ctx
        n_ff, k, n_out = 1024, 512, 192
        rg, ru = synth.random_weight(Q4_K, n_ff, k, seed=1), synth.random_weight(Q4_K, n_ff, k, seed=2)
        rd = synth.random_weight(Q6_K, n_out, n_ff, seed=3)
        ws = [g.upload(Q4_K, n_ff, k, rg, capi.LAYOUT_TILED), g.upload(Q4_K, n_ff, k, ru, capi.LAYOUT_TILED),
              g.upload(Q6_K, n_out, n_ff, rd, capi.LAYOUT_TILED)]
        x = synth.random_activation(m, k, seed=m, bf16=True) * np.float32(16.0)
        h = onp.silu_mul(orc.matmul_dequant(Q4_K, x, rg, n_ff, k), orc.matmul_dequant(Q4_K, x, ru, n_ff, k))
        assert np.abs(h).max() > 65520 and np.all(np.isfinite(h.astype(np.float32)))      # the case this test is about
        want = orc.matmul_dequant(Q6_K, h.astype(np.float32), rd, n_out, n_ff)
        nonfinite(g)
        y = g.mlp(*ws, x, n_ff, k, n_out)
        assert not np.all(np.isfinite(y))
        assert nonfinite(g) > 0
        capi.check(L.turq_ctx_set_wide_activations(ctx, 1), ctx)
        y = g.mlp(*ws, x, n_ff, k, n_out)
        assert np.all(np.isfinite(y))
        # (two matmuls in a row, each inside its own 1e-3: more than 32 rows go through the prefill GEMM, about 3e-4 a stage,
        # on an intermediate of six orders of magnitude)
        assert per_row_rel(y, want).max() <= (1e-3 if m <= 32 else 2e-3)
        assert nonfinite(g) == 0
        for w in ws:
            g.release(w)
    finally:
        g.close()
