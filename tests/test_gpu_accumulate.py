"""TURQ_OUT_ACCUMULATE: y += x * W^T (+ bias), the residual connection of the reference's decoder layer (`x + h` after o_proj,
`x + h2` after the MLP, src/models/qwen3.rs:633-640) taken into the store of the matmul kernels.

The sum is formed in f32 and rounded once to y's type, so the expected value is exact: the f32 result of the same call
without the flag, plus what y held, rounded like y.  Every kernel family is driven through the C ABI (one row, a few rows,
rows staged in the kernel, prepared fragments, the prefill GEMM with and without split columns, the dense and native-layout
kernel, host pointers, wide activations, turq_mlp, turq_qmatmul_noalloc)."""
import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu, rel_l2
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
ACC = 0x100
NP_OUT = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def to_type(v, yt):
    """f32 values rounded once to the output type, as the kernels store them; returned as f32"""
    v = np.asarray(v, np.float32)
    if yt == capi.ACT_BF16:
        return synth.from_bf16_bits(synth.to_bf16_bits(v)).reshape(v.shape)
    if yt == capi.ACT_F16:
        return v.astype(np.float16).astype(np.float32)
    return v


def as_stored(v, yt):
    v = np.asarray(v, np.float32)
    if yt == capi.ACT_BF16:
        return synth.to_bf16_bits(v).reshape(v.shape)
    return v.astype(NP_OUT[yt])


def widen(a, yt):
    if yt == capi.ACT_BF16:
        return synth.from_bf16_bits(a).reshape(a.shape)
    return np.asarray(a, np.float32)


def run(gpu, w, x, n, k, y0, yt, flag, bias=None, noalloc=False, mem=capi.MEM_DEVICE, x_dtype=capi.ACT_F32):
    """one turq_qmatmul on an output buffer that starts as y0 (values already representable in yt); returns f32 values"""
    L, ctx = gpu.L, gpu.ctx
    m = x.shape[0]
    xs = synth.to_bf16_bits(x).reshape(m, k) if x_dtype == capi.ACT_BF16 else np.ascontiguousarray(x, np.float32)
    ybuf = np.ascontiguousarray(as_stored(y0, yt))
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    if mem == capi.MEM_HOST:
        capi.check(L.turq_qmatmul(ctx, w, capi.ptr(xs), x_dtype, m, k, capi.ptr(ybuf), yt | flag, n, capi.ptr(b), mem, capi.ALGO_AUTO), ctx)
        return widen(ybuf, yt)
    xd, yd = gpu.dev_buffer(xs), gpu.dev_buffer(ybuf)
    bd = None if b is None else gpu.dev_buffer(b)
    try:
        if noalloc:
            capi.check(L.turq_qmatmul_noalloc(ctx, w, xd, x_dtype, m, k, yd, yt | flag, n, bd), ctx)
        else:
            capi.check(L.turq_qmatmul(ctx, w, xd, x_dtype, m, k, yd, yt | flag, n, bd, mem, capi.ALGO_AUTO), ctx)
        out = gpu.read_back(yd, (m, n), NP_OUT[yt])
    finally:
        for p in (xd, yd, bd):
            if p is not None:
                gpu.dev_free(p)
    return widen(out, yt)


CASES = [  # dtype, n, k, rows
    (Q4_K, 4096, 4096, (1, 2, 4, 8, 24)),       # one-row kernel (1, 2, 4 rows), rows staged in the kernel
    (Q6_K, 1040, 12288, (1, 3, 20, 32)),        # tall: prepared fragments at 17 .. 32 rows
    (Q8_0, 200, 1056, (1, 5, 40)),              # ragged Q8_0 columns: the skinny kernel in chunks at 40 rows
    (Q4_K, 512, 8192, (70, 128)),               # prefill GEMM with its columns split over workgroups
    (Q5_K, 1000, 2048, (33, 300)),              # prefill GEMM, ragged n (scalar stores) ...
    (Q6_K, 1024, 2048, (512,)),                 # ... and aligned (16-byte stores)
]


@pytest.mark.parametrize("yt", [capi.ACT_F32, capi.ACT_BF16, capi.ACT_F16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("dt,n,k,ms", CASES, ids=[f"{c[0]}-{c[1]}x{c[2]}" for c in CASES])
def test_results_are_added_to_the_output(gpu, dt, n, k, ms, yt):
    raw = synth.random_weight(dt, n, k, seed=n + k)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    rng = np.random.default_rng(n)
    bias = rng.standard_normal(n).astype(np.float32)
    for m in ms:
        x = synth.random_activation(m, k, seed=m, bf16=True)
        y0 = to_type(rng.standard_normal((m, n)).astype(np.float32) * 50.0, yt)
        plain = run(gpu, w, x, n, k, np.zeros((m, n), np.float32), capi.ACT_F32, 0, bias=bias, x_dtype=capi.ACT_BF16)
        assert rel_l2(plain, orc.matmul_dequant(dt, x, raw, n, k) + bias) <= 1e-3
        got = run(gpu, w, x, n, k, y0, yt, ACC, bias=bias, x_dtype=capi.ACT_BF16)
        want = to_type(plain + y0, yt)
        assert np.array_equal(got, want), (m, np.abs(got - want).max())
        # without the flag the buffer's contents do not matter
        assert np.array_equal(run(gpu, w, x, n, k, y0, yt, 0, bias=bias, x_dtype=capi.ACT_BF16), to_type(plain, yt)), m
    gpu.release(w)


def test_other_routes(gpu):
    """native layout, a dense F16 weight, host pointers, wide activations on device pointers, the call that allocates nothing"""
    dt, n, k = Q4_K, 320, 1024
    raw = synth.random_weight(dt, n, k, seed=5)
    rng = np.random.default_rng(1)
    for m in (1, 6, 48):
        x = synth.random_activation(m, k, seed=m)
        y0 = rng.standard_normal((m, n)).astype(np.float32)
        for layout in (capi.LAYOUT_NATIVE, capi.LAYOUT_TILED):
            w = gpu.upload(dt, n, k, raw, layout)
            plain = run(gpu, w, x, n, k, y0 * 0, capi.ACT_F32, 0)
            assert np.array_equal(run(gpu, w, x, n, k, y0, capi.ACT_F32, ACC), plain + y0)
            if layout == capi.LAYOUT_TILED:
                assert np.array_equal(run(gpu, w, x, n, k, y0, capi.ACT_F32, ACC, noalloc=True), plain + y0)
                # host pointers take the wide path (rows scaled into the f16 range): its own result plus the rows
                host_plain = run(gpu, w, x, n, k, y0 * 0, capi.ACT_F32, 0, mem=capi.MEM_HOST)
                assert np.array_equal(run(gpu, w, x, n, k, y0, capi.ACT_F32, ACC, mem=capi.MEM_HOST), host_plain + y0)
                capi.check(gpu.L.turq_ctx_set_wide_activations(gpu.ctx, 1), gpu.ctx)
                try:
                    big = x * np.float32(1e6)
                    wide_plain = run(gpu, w, big, n, k, y0 * 0, capi.ACT_F32, 0)
                    assert rel_l2(wide_plain, orc.matmul_dequant(dt, big, raw, n, k)) <= 1e-3
                    assert np.array_equal(run(gpu, w, big, n, k, y0, capi.ACT_F32, ACC), wide_plain + y0)
                    yb = to_type(y0, capi.ACT_BF16)
                    assert np.array_equal(run(gpu, w, big, n, k, yb, capi.ACT_BF16, ACC), to_type(wide_plain + yb, capi.ACT_BF16))
                finally:
                    capi.check(gpu.L.turq_ctx_set_wide_activations(gpu.ctx, 0), gpu.ctx)
            gpu.release(w)
    dense = rng.standard_normal((n, k)).astype(np.float16)
    w = gpu.upload(capi.F16, n, k, dense.view(np.uint8).reshape(-1), capi.LAYOUT_NATIVE)
    x = synth.random_activation(3, k, seed=9)
    y0 = rng.standard_normal((3, n)).astype(np.float32)
    plain = run(gpu, w, x, n, k, y0 * 0, capi.ACT_F32, 0)
    assert rel_l2(plain, x @ dense.astype(np.float32).T) <= 1e-5
    assert np.array_equal(run(gpu, w, x, n, k, y0, capi.ACT_F32, ACC), plain + y0)
    gpu.release(w)


@pytest.mark.parametrize("m", [1, 8, 32, 64, 200])
def test_mlp_adds_to_the_residual_stream(gpu, m):
    """turq_mlp with the flag: x + mlp(norm(x)) of the decoder layer in one call (the second residual of qwen3.rs:633-640)"""
    n_ff, k, n_out = 2048, 1024, 1024
    raws = [synth.random_weight(Q4_K, n_ff, k, seed=1), synth.random_weight(Q4_K, n_ff, k, seed=2), synth.random_weight(Q6_K, n_out, n_ff, seed=3)]
    ws = [gpu.upload(Q4_K, n_ff, k, raws[0], capi.LAYOUT_TILED), gpu.upload(Q4_K, n_ff, k, raws[1], capi.LAYOUT_TILED),
          gpu.upload(Q6_K, n_out, n_ff, raws[2], capi.LAYOUT_TILED)]
    L, ctx = gpu.L, gpu.ctx
    x = synth.random_activation(m, k, seed=m, bf16=True) * np.float32(0.01)
    y0 = np.random.default_rng(m).standard_normal((m, n_out)).astype(np.float32)
    plain = gpu.mlp(*ws, x, n_ff, k, n_out, x_dtype=capi.ACT_BF16)
    xd, yd = gpu.dev_buffer(synth.to_bf16_bits(x).reshape(m, k)), gpu.dev_buffer(y0)
    capi.check(L.turq_mlp(ctx, ws[0], ws[1], ws[2], xd, capi.ACT_BF16, m, k, yd, capi.ACT_F32 | ACC, n_out, None, None, None, 0, capi.MEM_DEVICE), ctx)
    got = gpu.read_back(yd, (m, n_out), np.float32)
    assert np.array_equal(got, plain + y0)
    gpu.dev_free(xd)
    gpu.dev_free(yd)
    for w in ws:
        gpu.release(w)


def test_the_flag_belongs_to_qmatmul_and_mlp(gpu):
    L, ctx = gpu.L, gpu.ctx
    raw = synth.random_weight(Q4_K, 64, 256, seed=1)
    w = gpu.upload(Q4_K, 64, 256, raw, capi.LAYOUT_TILED)
    x = np.zeros((1, 256), np.float32)
    y = np.zeros((1, 64), np.float32)
    warr = (ctypes.c_void_p * 1)(w.value)
    yarr = (ctypes.c_void_p * 1)(y.ctypes.data)
    ldys = (ctypes.c_int64 * 1)(64)
    assert L.turq_qmatmul_multi(ctx, 1, warr, capi.ptr(x), capi.ACT_F32, 1, 256, yarr, capi.ACT_F32 | ACC, ldys, None, capi.MEM_HOST, capi.ALGO_AUTO) == capi.ERR_DTYPE
    assert L.turq_qmatmul_gate_up(ctx, w, w, capi.ptr(x), capi.ACT_F32, 1, 256, capi.ptr(y), capi.ACT_F32 | ACC, 64, None, None, 0, capi.MEM_HOST) == capi.ERR_DTYPE
    assert L.turq_qmatmul(ctx, w, capi.ptr(x), capi.ACT_F32 | ACC, 1, 256, capi.ptr(y), capi.ACT_F32, 64, None, capi.MEM_HOST, capi.ALGO_AUTO) == capi.ERR_DTYPE
    assert L.turq_qmatmul(ctx, w, capi.ptr(x), capi.ACT_F32, 1, 256, capi.ptr(y), capi.ACT_F32 | 0x200, 64, None, capi.MEM_HOST, capi.ALGO_AUTO) == capi.ERR_DTYPE
    assert L.turq_qmatmul(ctx, w, capi.ptr(x), capi.ACT_F32, 1, 256, capi.ptr(y), capi.ACT_F32 | ACC, 64, None, capi.MEM_HOST, capi.ALGO_AUTO) == capi.OK
    gpu.release(w)
