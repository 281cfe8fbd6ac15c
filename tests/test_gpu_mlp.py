"""GPU parity of turq_mlp: down(act(gate(x)) * up(x)), the reference's whole MLP (src/models/qwen3.rs:161-167,
src/models/granite_41.rs:151-155), called through the C ABI.

The contract is "the results of turq_qmatmul_gate_up into f32 followed by turq_qmatmul, bit for bit"; both are checked against
the oracle's matmuls on dequantized weights with the oracle's SiLU product in between (bar 1e-3).
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
# the synthetic weights give products of a few hundred at unit activations, and their product would leave the f16 range that the
# second matmul rounds its input to; real MLPs sit far below that
XS = 0.01


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def f16_round(x):
    return x.astype(np.float16).astype(np.float32)


def expected(dt_gu, dt_dn, x, raw_g, raw_u, raw_d, n_ff, k, n_out, biases=(None, None, None)):
    g = orc.matmul_dequant(dt_gu, x, raw_g, n_ff, k)
    u = orc.matmul_dequant(dt_gu, x, raw_u, n_ff, k)
    if biases[0] is not None:
        g = g + biases[0]
    if biases[1] is not None:
        u = u + biases[1]
    h = onp.silu_mul(g, u)
    y = orc.matmul_dequant(dt_dn, f16_round(h), raw_d, n_out, n_ff)
    return y if biases[2] is None else y + biases[2]


def weights(gpu, dt_gu, dt_dn, n_ff, k, n_out, seed=1, layout=capi.LAYOUT_TILED):
    raws = [synth.random_weight(dt_gu, n_ff, k, seed=seed), synth.random_weight(dt_gu, n_ff, k, seed=seed + 1),
            synth.random_weight(dt_dn, n_out, n_ff, seed=seed + 2)]
    ws = [gpu.upload(dt_gu, n_ff, k, raws[0], layout), gpu.upload(dt_gu, n_ff, k, raws[1], layout),
          gpu.upload(dt_dn, n_out, n_ff, raws[2], layout)]
    return raws, ws


def two_calls(gpu, ws, x, n_ff, k, n_out, x_dtype=capi.ACT_F32, biases=(None, None, None)):
    h = gpu.gate_up(ws[0], ws[1], x, n_ff, k, x_dtype=x_dtype, bias_gate=biases[0], bias_up=biases[1])
    return gpu.qmatmul(ws[2], h, n_out, n_ff, bias=biases[2])


@pytest.mark.parametrize("dt_gu,dt_dn", [(Q4_K, Q4_K), (Q4_K, Q6_K)])
@pytest.mark.parametrize("x_dtype", [capi.ACT_F32, capi.ACT_BF16, capi.ACT_F16])
def test_one_row_equals_the_two_calls(gpu, dt_gu, dt_dn, x_dtype):
    # the MLP of Qwen3-8B at two thirds of its width
    n_ff, k, n_out = 8192, 4096, 4096
    raws, ws = weights(gpu, dt_gu, dt_dn, n_ff, k, n_out, seed=3)
    rng = np.random.default_rng(5)
    biases = tuple(rng.standard_normal(n).astype(np.float32) * 0.1 for n in (n_ff, n_ff, n_out))
    for trial, bs in enumerate([(None, None, None), biases]):
        x = synth.random_activation(1, k, seed=30 + trial) * XS
        if x_dtype == capi.ACT_BF16:
            x = synth.from_bf16_bits(synth.to_bf16_bits(x)).reshape(1, k)
        elif x_dtype == capi.ACT_F16:
            x = f16_round(x)
        launches = []
        y = gpu.mlp(*ws, x, n_ff, k, n_out, x_dtype=x_dtype, biases=bs, launches=launches)
        assert launches == [2], launches
        assert np.isfinite(y).all() and np.abs(y).max() > 0
        assert np.array_equal(y, two_calls(gpu, ws, x, n_ff, k, n_out, x_dtype=x_dtype, biases=bs))
        want = expected(dt_gu, dt_dn, f16_round(x), *raws, n_ff, k, n_out, biases=bs)
        assert rel_l2(y, want) <= 1e-4, rel_l2(y, want)
    for w in ws:
        gpu.release(w)


def test_calls_in_a_row_and_output_dtypes(gpu):
    # different inputs and output types, one call after the other
    n_ff, k, n_out = 8192, 4096, 2048
    raws, ws = weights(gpu, Q4_K, Q4_K, n_ff, k, n_out, seed=7)
    for i in range(6):
        x = synth.random_activation(1, k, seed=50 + i) * (XS * (0.2 + 0.05 * i))
        y_dtype = [capi.ACT_F32, capi.ACT_BF16, capi.ACT_F16][i % 3]
        launches = []
        y = gpu.mlp(*ws, x, n_ff, k, n_out, y_dtype=y_dtype, launches=launches)
        assert launches == [2]
        want = expected(Q4_K, Q4_K, f16_round(x), *raws, n_ff, k, n_out)
        assert rel_l2(y, want) <= (1e-4 if y_dtype == capi.ACT_F32 else 4e-3 if y_dtype == capi.ACT_BF16 else 6e-4)
    for w in ws:
        gpu.release(w)


@pytest.mark.parametrize("dt_gu,dt_dn", [(Q8_0, Q8_0), (Q5_K, Q6_K), (Q6_K, Q6_K), (Q4_K, Q4_K)])
@pytest.mark.parametrize("m", [0, 1, 2, 5, 40])
def test_every_other_case_is_the_two_calls(gpu, dt_gu, dt_dn, m):
    # small or ragged shapes, several rows, every format
    n_ff, k, n_out = 768, 512 + (32 if dt_gu == Q8_0 else 0), 200
    raws, ws = weights(gpu, dt_gu, dt_dn, n_ff, k, n_out, seed=11)
    x = synth.random_activation(m, k, seed=m + 1) * XS
    y = gpu.mlp(*ws, x, n_ff, k, n_out)
    assert y.shape == (m, n_out)
    if m:
        assert np.array_equal(y, two_calls(gpu, ws, x, n_ff, k, n_out))
        want = expected(dt_gu, dt_dn, f16_round(x), *raws, n_ff, k, n_out)
        assert rel_l2(y, want) <= 1e-3, rel_l2(y, want)
    for w in ws:
        gpu.release(w)


def test_host_pointers_and_native_layout(gpu):
    n_ff, k, n_out = 512, 256, 96
    raws, ws = weights(gpu, Q4_K, Q6_K, n_ff, k, n_out, seed=13, layout=capi.LAYOUT_NATIVE)
    x = synth.random_activation(3, k, seed=4) * XS
    want = expected(Q4_K, Q6_K, x, *raws, n_ff, k, n_out)
    assert rel_l2(gpu.mlp(*ws, x, n_ff, k, n_out, mem=capi.MEM_HOST), want) <= 1e-3
    assert rel_l2(gpu.mlp(*ws, x, n_ff, k, n_out), want) <= 1e-3
    for w in ws:
        gpu.release(w)


def test_argument_errors(gpu):
    raws, ws = weights(gpu, Q4_K, Q4_K, 512, 256, 64, seed=17)
    wrong = gpu.upload(Q4_K, 64, 256, synth.random_weight(Q4_K, 64, 256, seed=1), capi.LAYOUT_TILED)
    x = np.zeros((1, 256), np.float32)
    y = np.zeros((1, 64), np.float32)
    L = gpu.L
    call = lambda g, u, d, act=0, mem=capi.MEM_HOST, yt=capi.ACT_F32: L.turq_mlp(gpu.ctx, g, u, d, capi.ptr(x), capi.ACT_F32, 1, 256, capi.ptr(y), yt, 64, None, None, None, act, mem)
    assert call(ws[0], ws[1], ws[2]) == capi.OK
    assert call(None, ws[1], ws[2]) == capi.ERR_INVALID
    assert call(ws[0], ws[1], wrong) == capi.ERR_SHAPE and b"down takes 256 columns" in L.turq_last_error(gpu.ctx)
    assert call(ws[0], wrong, ws[2]) == capi.ERR_SHAPE
    assert call(ws[0], ws[1], ws[2], act=3) == capi.ERR_INVALID
    assert call(ws[0], ws[1], ws[2], mem=7) == capi.ERR_INVALID
    assert call(ws[0], ws[1], ws[2], yt=9) == capi.ERR_DTYPE
    for w in ws + [wrong]:
        gpu.release(w)


def test_inside_a_graph(gpu):
    # three MLP calls back to back (the same input: chained, the synthetic weights would leave the f16 range), captured once and
    # replayed with eager work in between
    n_ff, k, n_out = 8192, 4096, 4096
    raws, ws = weights(gpu, Q4_K, Q6_K, n_ff, k, n_out, seed=19)
    L, ctx = gpu.L, gpu.ctx
    x0 = synth.random_activation(1, k, seed=9) * XS
    bufs = [gpu.dev_buffer(x0)] + [gpu.dev_buffer(np.zeros((1, n_out), np.float32)) for _ in range(3)]

    def chain():
        for i in range(3):
            capi.check(L.turq_mlp(ctx, ws[0], ws[1], ws[2], bufs[0], capi.ACT_F32, 1, k, bufs[i + 1], capi.ACT_F32, n_out, None, None, None,
                                  0, capi.MEM_DEVICE), ctx)

    chain()
    capi.check(L.turq_sync(ctx), ctx)
    eager = gpu.read_back(bufs[3], (1, n_out), np.float32)
    assert np.isfinite(eager).all() and np.abs(eager).max() > 0
    assert rel_l2(eager, expected(Q4_K, Q6_K, f16_round(x0), *raws, n_ff, k, n_out)) <= 1e-4
    capi.check(L.turq_graph_begin(ctx), ctx)
    chain()
    g = ctypes.c_void_p()
    capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
    for rep in range(4):
        for b in bufs[1:]:
            capi.check(L.turq_memcpy_h2d(ctx, b, capi.ptr(np.zeros((1, n_out), np.float32)), 4 * n_out), ctx)
        capi.check(L.turq_graph_launch(ctx, g), ctx)
        capi.check(L.turq_sync(ctx), ctx)
        for b in bufs[1:]:
            assert np.array_equal(gpu.read_back(b, (1, n_out), np.float32), eager), rep
        gpu.mlp(*ws, synth.random_activation(1, k, seed=100 + rep) * XS, n_ff, k, n_out)  # eager work between the replays
    L.turq_graph_destroy(g)
    for b in bufs:
        gpu.dev_free(b)
    for w in ws:
        gpu.release(w)


@pytest.mark.parametrize("dt_gu,dt_dn", [(Q4_K, Q6_K), (Q5_K, Q4_K)])
@pytest.mark.parametrize("m", [72, 128, 512])
def test_prompt_chunks(gpu, dt_gu, dt_dn, m):
    """More than 32 rows: gate / up GEMMs into f32 scratch, ONE kernel from the two products to down_proj's fragments (no f16 copy
    of the intermediate, no separate preparation), down_proj's GEMM.  Bit-equal to the two calls, within 1e-3 of the oracle's
    chain; bf16 in and out as a prompt chunk has them, and with biases."""
    n_ff, k, n_out = 3072, 2048, 1536
    raws, ws = weights(gpu, dt_gu, dt_dn, n_ff, k, n_out, seed=23 + m)
    rng = np.random.default_rng(m)
    biases = tuple(rng.standard_normal(n).astype(np.float32) * 0.1 for n in (n_ff, n_ff, n_out))
    x = synth.random_activation(m, k, seed=m, bf16=True) * XS
    x = synth.from_bf16_bits(synth.to_bf16_bits(x)).reshape(m, k)
    for bs in ((None, None, None), biases):
        launches = []
        y = gpu.mlp(*ws, x, n_ff, k, n_out, x_dtype=capi.ACT_BF16, biases=bs, launches=launches)
        assert np.array_equal(y, two_calls(gpu, ws, x, n_ff, k, n_out, x_dtype=capi.ACT_BF16, biases=bs))
        g = orc.matmul_dequant(dt_gu, x, raws[0], n_ff, k) + (0 if bs[0] is None else bs[0])
        u = orc.matmul_dequant(dt_gu, x, raws[1], n_ff, k) + (0 if bs[1] is None else bs[1])
        want = orc.matmul_dequant(dt_dn, onp.silu_mul(g, u).astype(np.float32), raws[2], n_out, n_ff) + (0 if bs[2] is None else bs[2])
        assert rel_l2(y, want) <= 1e-3, rel_l2(y, want)
    yb = gpu.mlp(*ws, x, n_ff, k, n_out, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16, biases=biases)
    assert np.array_equal(synth.to_bf16_bits(yb).reshape(m, n_out), synth.to_bf16_bits(y).reshape(m, n_out))
    for w in ws:
        gpu.release(w)
