"""GPU parity of turq_qmatmul (the QMatMul::forward replacement), called through the C ABI.

Bars (relative L2 over the whole output):
  * <= 1e-3 against the f32 matmul on oracle-dequantized weights (f64-accumulated),
  * <= 1e-2 against the restated candle CPU QMatMul (which quantises activations to Q8_K / Q8_0),
and two sharper ones that catch indexing slips the loose bars could hide:
  * the plain kernel (f32 FMA on dequantized values) must agree to 2e-5,
  * the MFMA kernel must agree to 2e-5 once the oracle is given the same f16-rounded activations
    (its weight side is exact integer arithmetic).
"""
import ctypes

import numpy as np
import pytest

from oracle import capi as orc
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


def check_all_bars(y, dt, x, raw, n, k, f16_acts, sharp_bar=2e-5):
    dense = orc.matmul_dequant(dt, x, raw, n, k)
    assert rel_l2(y, dense) <= 1e-3
    cpu = orc.qmatmul(dt, x, raw, n, k)
    assert rel_l2(y, cpu) <= 1e-2
    sharp = orc.matmul_dequant(dt, f16_round(x), raw, n, k) if f16_acts else dense
    assert rel_l2(y, sharp) <= sharp_bar, rel_l2(y, sharp)


@pytest.mark.parametrize("dt", ALL)
@pytest.mark.parametrize("m", [1, 5])
def test_simple_kernel_native_layout(gpu, dt, m):
    n, k = 77, 1024
    raw = synth.random_weight(dt, n, k, seed=dt * 3 + m)
    x = synth.random_activation(m, k, seed=m)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_NATIVE)
    y = gpu.qmatmul(w, x, n, k, algo=capi.ALGO_SIMPLE)
    gpu.release(w)
    check_all_bars(y, dt, x, raw, n, k, f16_acts=False)


@pytest.mark.parametrize("dt", ALL)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 13, 16, 17, 32])
def test_mfma_gemv_tiled_layout(gpu, dt, m):
    n, k = 200, 2048           # ragged row tile (200 = 12 * 16 + 8), 8 column tiles
    raw = synth.random_weight(dt, n, k, seed=dt * 5 + m)
    x = synth.random_activation(m, k, seed=m + 50)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    y = gpu.qmatmul(w, x, n, k, algo=capi.ALGO_GEMV)
    gpu.release(w)
    check_all_bars(y, dt, x, raw, n, k, f16_acts=True)


@pytest.mark.parametrize("dt", ALL)
def test_mfma_more_rows_than_one_launch(gpu, dt):
    n, k, m = 64, 512, 70       # m > 32: the GEMM kernel
    raw = synth.random_weight(dt, n, k, seed=dt)
    x = synth.random_activation(m, k, seed=70)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    y = gpu.qmatmul(w, x, n, k)
    gpu.release(w)
    # the GEMM folds the f16 block scale into its f16 weights: 2 - 3e-4 instead of exact integers
    check_all_bars(y, dt, x, raw, n, k, f16_acts=True, sharp_bar=4e-4)


@pytest.mark.parametrize("dt", ALL)
def test_single_tile_shapes(gpu, dt):
    # the smallest legal shapes: one block of columns, one row
    k = 256
    for n in (1, 16, 17):
        raw = synth.random_weight(dt, n, k, seed=n)
        x = synth.random_activation(2, k, seed=n + 1)
        for layout, sharp in ((capi.LAYOUT_NATIVE, False), (capi.LAYOUT_TILED, True)):
            w = gpu.upload(dt, n, k, raw, layout)
            y = gpu.qmatmul(w, x, n, k)
            gpu.release(w)
            ref = orc.matmul_dequant(dt, f16_round(x) if sharp else x, raw, n, k)
            assert rel_l2(y, ref) <= 2e-5


def test_q8_0_ragged_k(gpu):
    # Q8_0 needs k % 32 == 0 only: 96 columns fill 3 of the 8 blocks of a column tile
    n, k = 48, 96 + 256
    raw = synth.random_weight(Q8_0, n, k, seed=4)
    x = synth.random_activation(3, k, seed=5)
    w = gpu.upload(Q8_0, n, k, raw, capi.LAYOUT_TILED)
    y = gpu.qmatmul(w, x, n, k)
    gpu.release(w)
    assert rel_l2(y, orc.matmul_dequant(Q8_0, f16_round(x), raw, n, k)) <= 2e-5


@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED])
def test_activation_and_output_dtypes(gpu, layout):
    n, k, m = 96, 1024, 4
    raw = synth.random_weight(Q4_K, n, k, seed=21)
    x = synth.random_activation(m, k, seed=22, bf16=True)     # bf16-representable values
    w = gpu.upload(Q4_K, n, k, raw, layout)
    dense = orc.matmul_dequant(Q4_K, x, raw, n, k)
    # bf16 activations are exact in both kernels (bf16 -> f16 loses nothing for |x| in the f16 range)
    y = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16)
    assert rel_l2(y, dense) <= 2e-5
    y = gpu.qmatmul(w, x.astype(np.float16).astype(np.float32), n, k, x_dtype=capi.ACT_F16)
    assert rel_l2(y, orc.matmul_dequant(Q4_K, f16_round(x), raw, n, k)) <= 2e-5
    # bf16 store: compare with the oracle rounded the same way (round to nearest even)
    yb = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16)
    want = synth.from_bf16_bits(synth.to_bf16_bits(dense)).reshape(m, n)
    assert rel_l2(yb, want) <= 2e-3 and rel_l2(yb, dense) <= 4e-3
    yh = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_F16)
    assert rel_l2(yh, dense) <= 5e-4
    gpu.release(w)


@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED])
def test_bias_and_row_strides(gpu, layout):
    n, k, m = 50, 512, 3
    raw = synth.random_weight(Q6_K, n, k, seed=31)
    x = synth.random_activation(m, k, seed=32, bf16=True)
    bias = np.random.default_rng(33).standard_normal(n).astype(np.float32)
    w = gpu.upload(Q6_K, n, k, raw, layout)
    y = gpu.qmatmul(w, x, n, k, bias=bias, ldx=k + 24, ldy=n + 7)
    gpu.release(w)
    want = orc.matmul_dequant(Q6_K, x, raw, n, k) + bias[None, :]
    assert rel_l2(y, want) <= 2e-5


def test_linearity_and_zero_input(gpu):
    # size-independent properties at a full Qwen3-8B row count: f(0) = 0, f(2x) = 2 f(x) exactly
    # (scaling by 2 is exact in f16 and f32), f(x1 + x2) ~= f(x1) + f(x2)
    n, k = 4096, 4096
    raw = synth.random_weight(Q4_K, n, k, seed=41)
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_TILED)
    x1 = synth.random_activation(1, k, seed=42, bf16=True)
    x2 = synth.random_activation(1, k, seed=43, bf16=True)
    y0 = gpu.qmatmul(w, np.zeros((1, k), np.float32), n, k)
    assert np.all(y0 == 0)
    y1 = gpu.qmatmul(w, x1, n, k)
    assert np.array_equal(gpu.qmatmul(w, 2 * x1, n, k), 2 * y1)
    y2 = gpu.qmatmul(w, x2, n, k)
    y12 = gpu.qmatmul(w, x1 + x2, n, k)
    assert rel_l2(y12, y1 + y2) <= 1e-3
    gpu.release(w)


def test_weight_clone_shares_device_copy(gpu):
    # Arc<QTensor> semantics: retain / release, the weight stays usable until the last release
    n, k = 32, 256
    raw = synth.random_weight(Q4_K, n, k, seed=51)
    x = synth.random_activation(1, k, seed=52)
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_TILED)
    capi.check(gpu.L.turq_weight_retain(w))
    gpu.release(w)
    y = gpu.qmatmul(w, x, n, k)
    gpu.release(w)
    assert rel_l2(y, orc.matmul_dequant(Q4_K, f16_round(x), raw, n, k)) <= 2e-5


def test_error_paths(gpu):
    L, ctx = gpu.L, gpu.ctx
    n, k = 32, 256
    raw = synth.random_weight(Q4_K, n, k, seed=61)
    import ctypes
    w = ctypes.c_void_p()
    # wrong byte count, k not a multiple of the block, unknown dtype
    assert L.turq_weight_upload(ctx, Q4_K, n, k, capi.ptr(raw), raw.size - 1, 0, ctypes.byref(w)) == capi.ERR_SHAPE
    assert "bytes" in capi.last_error(ctx)
    assert L.turq_weight_upload(ctx, Q4_K, n, 100, capi.ptr(raw), raw.size, 0, ctypes.byref(w)) == capi.ERR_SHAPE
    assert L.turq_weight_upload(ctx, 99, n, k, capi.ptr(raw), raw.size, 0, ctypes.byref(w)) == capi.ERR_DTYPE
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_TILED)
    x = np.zeros((2, k), np.float32)
    y = np.zeros((2, n), np.float32)
    call = lambda **kw: L.turq_qmatmul(ctx, w, capi.ptr(x), kw.get("xt", 0), kw.get("m", 2), kw.get("ldx", k), capi.ptr(y),
                                       kw.get("yt", 0), kw.get("ldy", n), None, kw.get("mem", 0), kw.get("algo", 0))
    assert call(ldx=k - 1) == capi.ERR_SHAPE            # last dim != k
    assert call(ldy=n - 1) == capi.ERR_SHAPE
    assert call(m=-1) == capi.ERR_SHAPE
    assert call(xt=7) == capi.ERR_DTYPE
    assert call(algo=capi.ALGO_SIMPLE) == capi.ERR_INVALID   # plain kernel needs the native layout
    assert call(m=0) == capi.OK                          # empty batch is a no-op
    assert call() == capi.OK
    gpu.release(w)


# ---------------------------------------------------------------------------------------------
# prefill GEMM (m > 32): weights carry the f16 product d * sc (Q8_0: q * d) inside the kernel, so the
# sharp bar is looser than the GEMV's; the 1e-3 bar against the f32 matmul on dequantized weights holds
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", [Q4_K, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("n,k,m", [(96, 256, 33), (200, 1024, 300), (512, 2048, 512), (100, 512, 700), (16, 768, 129)])
def test_prefill_gemm(gpu, dt, n, k, m):
    raw = synth.random_weight(dt, n, k, seed=n + m)
    x = synth.random_activation(m, k, seed=m, bf16=True)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    dense = orc.matmul_dequant(dt, x, raw, n, k)
    y = gpu.qmatmul(w, x, n, k, algo=capi.ALGO_GEMM, x_dtype=capi.ACT_BF16)
    assert rel_l2(y, dense) <= 1e-3
    assert rel_l2(y, dense) <= 4e-4, rel_l2(y, dense)           # what the folded f16 scales are expected to cost
    yg = gpu.qmatmul(w, x, n, k, algo=capi.ALGO_GEMV, x_dtype=capi.ACT_BF16)   # same call through the chunked skinny kernel
    assert rel_l2(yg, dense) <= 2e-5                            # (which keeps the weights as exact integers)
    assert rel_l2(y, yg) <= 5e-4
    # bf16 store, compared with the oracle rounded the same way; bias rides along
    bias = np.random.default_rng(1).standard_normal(n).astype(np.float32)
    yb = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16, bias=bias, ldx=k + 8, ldy=n + 3)
    want = synth.from_bf16_bits(synth.to_bf16_bits(dense + bias)).reshape(m, n)
    assert rel_l2(yb, want) <= 3e-3 and rel_l2(yb, dense + bias) <= 4e-3
    # row strides that keep 16-byte alignment leave through the wide stores (when n is a multiple of 8), f16 and bf16
    for yd, bar in ((capi.ACT_F16, 1.2e-3), (capi.ACT_BF16, 4e-3)):
        ya = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=yd, bias=bias, ldy=n + (-n) % 8 + 8)
        assert rel_l2(ya, dense + bias) <= bar
    # f32 activations take the same path (rounded to f16 on the way in)
    xf = synth.random_activation(m, k, seed=m + 1)
    yf = gpu.qmatmul(w, xf, n, k)
    assert rel_l2(yf, orc.matmul_dequant(dt, xf, raw, n, k)) <= 1e-3
    gpu.release(w)


@pytest.mark.parametrize("dt", [Q6_K, Q5_K])
def test_prefill_tall_weight_f32_and_bf16(gpu, dt):
    # a vocabulary-like weight (many rows, ragged) at 128 rows: the 128 x 128 tile of the 1 x 4 wave grid by the rule, the wide
    # 128 x 256 tile when test_prefill_tile_shapes forces it; f32 result against the oracle on every 8th row, and the bf16
    # output is that result rounded once, bit for bit
    n, k, m = 20000, 4096, 128
    raw = synth.random_weight(dt, n, k, seed=dt + 70)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    x = synth.random_activation(m, k, seed=71, bf16=True)
    y = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16)
    yb = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16)
    gpu.release(w)
    rows = np.arange(1, n, 8)
    sub = raw.reshape(n, -1)[rows].reshape(-1)
    assert np.all(np.isfinite(y))
    assert rel_l2(y[:, rows], orc.matmul_dequant(dt, x, sub, len(rows), k)) <= 1e-3
    assert np.array_equal(synth.to_bf16_bits(y).reshape(m, n), synth.to_bf16_bits(yb).reshape(m, n))



# Tall-k matrices at prefill chunk sizes (down_proj: 4096 x 12288) make few workgroup tiles, so the launcher gives every tile
# to several workgroups that each take a part of the columns and meet in device memory.  Shapes that split on a 256-CU device
# (few tiles, many super-blocks): results against the oracle, twice in a row (the tiles' counters must be back at zero), with
# bias, row strides, a ragged n and m, and every output type.
@pytest.mark.parametrize("dt", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("n,k,m", [(512, 8192, 128), (200, 6144, 70), (1024, 12288, 300), (256, 4096, 512)])
def test_prefill_gemm_split_columns(gpu, dt, n, k, m):
    raw = synth.random_weight(dt, n, k, seed=n + m)
    x = synth.random_activation(m, k, seed=m, bf16=True)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    dense = orc.matmul_dequant(dt, x, raw, n, k)
    y = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16)
    assert rel_l2(y, dense) <= 4e-4, rel_l2(y, dense)
    y2 = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16)
    assert np.array_equal(y, y2)                                # same sums in the same order on every launch
    bias = np.random.default_rng(2).standard_normal(n).astype(np.float32)
    yb = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16, bias=bias, ldx=k + 8, ldy=n + 3)
    assert rel_l2(yb, dense + bias) <= 4e-3
    ya = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_F16, bias=bias, ldy=n + (-n) % 8 + 8)
    assert rel_l2(ya, dense + bias) <= 1.2e-3
    # fewer rows right after: other tiles, other counters
    y3 = gpu.qmatmul(w, x[: m // 2 + 1], n, k, x_dtype=capi.ACT_BF16)
    assert rel_l2(y3, dense[: m // 2 + 1]) <= 4e-4
    gpu.release(w)


@pytest.mark.parametrize("dt", [Q4_K, Q5_K, Q6_K, Q8_0])
def test_prefill_gemm_large_scales_fall_back(gpu, dt):
    # (base + q) * d * sc would overflow f16 inside the GEMM: the dispatcher must take the exact skinny kernel instead
    n, k, m = 64, 512, 80
    bs = {Q4_K: 144, Q5_K: 176, Q6_K: 210, Q8_0: 34}[dt]
    raw = synth.random_weight(dt, n, k, seed=3).reshape(-1, bs)
    d_at = 208 if dt == Q6_K else 0
    big = 600.0 if dt == Q8_0 else 3.0     # d = 3 -> 1024 * 63 * d, 256 * 128 * d > 65504; Q8_0: 127 * 600 > 65504
    raw[:, d_at:d_at + 2] = np.array([big], np.float16).view(np.uint8)
    raw = raw.reshape(-1)
    x = synth.random_activation(m, k, seed=4, bf16=True)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    y = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16)
    gpu.release(w)
    assert np.all(np.isfinite(y))
    assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k)) <= 2e-5


@pytest.mark.parametrize("dt", [Q4_K, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("shrink", [1 / 300, 1 / 3000])
def test_prefill_gemm_small_scales(gpu, dt, shrink):
    # real checkpoints carry super-block scales around 1e-5 .. 1e-4, where d * sc (and d * sc / 16 of Q5_K) would sit in
    # the f16 subnormals: the GEMM multiplies the scales of a tensor by a power of two first and divides the result
    n, k, m = 256, 2048, 64
    bs = {Q4_K: 144, Q5_K: 176, Q6_K: 210, Q8_0: 34}[dt]
    x = synth.random_activation(m, k, seed=m, bf16=True)
    # Q4_K / Q5_K a second time with dmin left as it is: the power of two must leave room for dmin * m as well
    for fields in ([[208]] if dt == Q6_K else [[0]] if dt == Q8_0 else [[0, 2], [0]]):
        raw = synth.random_weight(dt, n, k, seed=5).reshape(-1, bs).copy()
        for at in fields:
            d = raw[:, at:at + 2].copy().view(np.float16).astype(np.float32) * np.float32(shrink)
            raw[:, at:at + 2] = d.astype(np.float16).view(np.uint8)
        raw = raw.reshape(-1)
        w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
        y = gpu.qmatmul(w, x, n, k, algo=capi.ALGO_GEMM, x_dtype=capi.ACT_BF16)
        gpu.release(w)
        assert np.all(np.isfinite(y))
        assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k)) <= 4e-4, fields


def test_prefill_q8_0_ragged_k_takes_the_skinny_kernel(gpu):
    # Q8_0 rows may end inside a 256-column tile; the GEMM wants whole tiles, so these shapes walk m in chunks
    n, k, m = 80, 256 + 96, 70
    raw = synth.random_weight(Q8_0, n, k, seed=11)
    x = synth.random_activation(m, k, seed=12, bf16=True)
    w = gpu.upload(Q8_0, n, k, raw, capi.LAYOUT_TILED)
    y = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16)
    gpu.release(w)
    assert rel_l2(y, orc.matmul_dequant(Q8_0, x, raw, n, k)) <= 2e-5


# ---------------------------------------------------------------------------------------------
# one activation row (decode): the kernel that applies the sub-block scales on the MFMA result
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ALL)
@pytest.mark.parametrize("n,k", [(1, 256), (17, 256), (200, 2048), (100, 12288), (48, 4096 + 256)])
def test_one_row(gpu, dt, n, k):
    if dt == Q8_0:
        k += 96                      # Q8_0 rows end inside a column tile
    raw = synth.random_weight(dt, n, k, seed=dt + n + k)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    rng = np.random.default_rng(n * 7 + k)
    base = synth.random_activation(1, k, seed=k + n)
    sparse = base * (rng.random((1, k)) < 0.05)
    cases = {
        "normal": (base, 2e-5),
        # no cancellation in sum(base * x): the accumulator starts 1024 * 32 * |x| away from the result
        "one-sided": (np.abs(base) + 3.0, 1e-4),
        "large": (base * 2000.0, 2e-5),
        "tiny": (base * 1e-3, 2e-5),
        "sparse": (sparse.astype(np.float32), 2e-5),
    }
    for name, (x, bar) in cases.items():
        want = orc.matmul_dequant(dt, f16_round(x), raw, n, k)
        y = gpu.qmatmul(w, x, n, k)
        assert rel_l2(y, want) <= bar, (name, rel_l2(y, want))
    # 16-bit activations and outputs, bias (errors measured against the product itself: a bias may cancel it)
    x = synth.random_activation(1, k, seed=3, bf16=True)
    bias = rng.standard_normal(n).astype(np.float32)
    prod = orc.matmul_dequant(dt, x, raw, n, k)

    def err(y, want):
        return float(np.linalg.norm(y - want) / np.linalg.norm(prod))

    assert err(gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, bias=bias), prod + bias) <= 2e-5
    assert err(gpu.qmatmul(w, f16_round(x), n, k, x_dtype=capi.ACT_F16, bias=bias),
               orc.matmul_dequant(dt, f16_round(x), raw, n, k) + bias) <= 2e-5
    yb = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16, bias=bias)
    assert rel_l2(yb, synth.from_bf16_bits(synth.to_bf16_bits(prod + bias)).reshape(1, n)) <= 2e-3
    assert rel_l2(gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_F16, bias=bias), prod + bias) <= 5e-4
    # the candle CPU path on the same input (its own activation quantisation is the difference: about 7e-3 once
    # there are enough blocks to average over, more on a single super-block)
    if k >= 2048:
        assert rel_l2(gpu.qmatmul(w, base, n, k), orc.qmatmul(dt, base, raw, n, k)) <= 1e-2
    gpu.release(w)


# ---------------------------------------------------------------------------------------------
# several weights against the same activations (q/k/v, gate/up): one launch per run of equal formats
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dts", [(Q4_K, Q4_K), (Q6_K, Q6_K, Q6_K), (Q8_0, Q8_0), (Q4_K, Q4_K, Q6_K), (Q5_K, Q5_K, Q6_K),
                                 (Q5_K, Q4_K, Q4_K, Q4_K, Q4_K, Q4_K)])
@pytest.mark.parametrize("m", [1, 3, 8, 20, 32])
def test_multi_weight_launch(gpu, dts, m):
    k = 1024
    ns = [64, 100, 272, 16, 48, 528][: len(dts)]
    raws = [synth.random_weight(dt, n, k, seed=10 * i + n) for i, (dt, n) in enumerate(zip(dts, ns))]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    x = synth.random_activation(m, k, seed=m, bf16=True)
    biases = [None if i == 1 else np.random.default_rng(i).standard_normal(n).astype(np.float32) for i, n in enumerate(ns)]
    for x_dtype in (capi.ACT_F32, capi.ACT_BF16):
        ys = gpu.qmatmul_multi(ws, x, ns, k, x_dtype=x_dtype, biases=biases)
        for dt, n, raw, w, y, b in zip(dts, ns, raws, ws, ys, biases):
            want = orc.matmul_dequant(dt, x, raw, n, k) + (0 if b is None else b)
            assert rel_l2(y, want) <= 2e-5, (dt, n)
            single = gpu.qmatmul(w, x, n, k, x_dtype=x_dtype, bias=b)
            assert rel_l2(y, single) <= 1e-6, (dt, n)     # same kernel body; only the split over waves may differ
    for w in ws:
        gpu.release(w)


@pytest.mark.parametrize("dts", [(Q4_K, Q6_K), (Q4_K, Q4_K, Q4_K, Q6_K), (Q4_K, Q6_K, Q6_K), (Q6_K, Q4_K), (Q4_K,) * 4 + (Q6_K,),
                                 (Q5_K, Q5_K, Q6_K), (Q5_K, Q6_K, Q6_K), (Q4_K, Q5_K, Q6_K)])
@pytest.mark.parametrize("k", [256, 4096, 12288])
def test_two_formats_in_one_row_launch(gpu, dts, k):
    # one activation row against Q4_K (or Q5_K) weights followed by Q6_K ones (q, k, v of a Q4_K_M / Q5_K_M file): one launch
    # when they are at most four; other orders and longer lists go out run by run.  Either way every result equals the single call.
    ns = [80, 16, 33, 272, 48][: len(dts)]
    raws = [synth.random_weight(dt, n, k, seed=7 * i + n + k) for i, (dt, n) in enumerate(zip(dts, ns))]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    x = synth.random_activation(1, k, seed=k, bf16=True)
    biases = [None if i == 0 else np.random.default_rng(i).standard_normal(n).astype(np.float32) for i, n in enumerate(ns)]
    for x_dtype in (capi.ACT_F32, capi.ACT_BF16):
        ys = gpu.qmatmul_multi(ws, x, ns, k, x_dtype=x_dtype, biases=biases)
        for dt, n, raw, w, y, b in zip(dts, ns, raws, ws, ys, biases):
            want = orc.matmul_dequant(dt, x, raw, n, k) + (0 if b is None else b)
            assert rel_l2(y, want) <= 2e-5, (dt, n)
            single = gpu.qmatmul(w, x, n, k, x_dtype=x_dtype, bias=b)
            assert np.array_equal(y, single), (dt, n)      # same kernel body, same split over waves
    for w in ws:
        gpu.release(w)


@pytest.mark.parametrize("dt", ALL)
def test_two_rows_on_a_large_weight(gpu, dt):
    # two activation rows on a weight of more than 8 MiB go through the one-row kernel's two-row form (no preparation launch);
    # smaller weights and more rows take the general kernel
    n, k = 4096, 4096 + (96 if dt == Q8_0 else 0)
    raw = synth.random_weight(dt, n, k, seed=dt)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    x = synth.random_activation(2, k, seed=5)
    bias = np.random.default_rng(2).standard_normal(n).astype(np.float32)
    y = gpu.qmatmul(w, x, n, k, bias=bias, ldx=k + 4, ldy=n + 5)
    want = orc.matmul_dequant(dt, f16_round(x), raw, n, k) + bias
    assert rel_l2(y, want) <= 2e-5
    for m in (1, 3):       # the rows are independent of each other: row i of any batch equals the one-row result
        ym = gpu.qmatmul(w, np.concatenate([x, x])[:m], n, k, bias=bias)
        assert rel_l2(ym, want[:1] if m == 1 else np.concatenate([want, want])[:m]) <= 2e-5
    xb = synth.random_activation(2, k, seed=6, bf16=True)
    yb = gpu.qmatmul(w, xb, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16)
    assert rel_l2(yb, orc.matmul_dequant(dt, xb, raw, n, k)) <= 4e-3      # bf16 store
    gpu.release(w)


@pytest.mark.parametrize("dt", ALL)
@pytest.mark.parametrize("m", [3, 4])
def test_up_to_four_rows_on_a_large_weight(gpu, dt, m):
    # Q4_K / Q5_K: pairs of activation rows share an MFMA chain in the one-row kernel (three rows: the fourth repeats the
    # first and is not stored); the other formats take the general kernel.  Distinct rows, strides, bias, every activation type.
    n, k = 4100, 4096 + (96 if dt == Q8_0 else 0)
    raw = synth.random_weight(dt, n, k, seed=dt + m)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    x = synth.random_activation(m, k, seed=11 + m)
    bias = np.random.default_rng(3).standard_normal(n).astype(np.float32)
    y = gpu.qmatmul(w, x, n, k, bias=bias, ldx=k + 8, ldy=n + 3)
    want = orc.matmul_dequant(dt, f16_round(x), raw, n, k) + bias
    assert y.shape == (m, n) and rel_l2(y, want) <= 2e-5
    for i in range(m):      # row i alone gives the same numbers up to the order of the sums
        assert rel_l2(gpu.qmatmul(w, x[i:i + 1], n, k, bias=bias), y[i:i + 1]) <= 1e-5, i
    xb = synth.random_activation(m, k, seed=21, bf16=True)
    yb = gpu.qmatmul(w, xb, n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_F32)
    assert rel_l2(yb, orc.matmul_dequant(dt, xb, raw, n, k)) <= 2e-5
    xh = f16_round(x)
    yh = gpu.qmatmul(w, xh, n, k, x_dtype=capi.ACT_F16, y_dtype=capi.ACT_F32)
    assert rel_l2(yh, want - bias) <= 2e-5
    gpu.release(w)


@pytest.mark.parametrize("dt", [Q4_K, Q5_K])
def test_four_rows_wide_weight(gpu, dt):
    # 48 column tiles: sixteen waves per workgroup, two tiles in flight and two pairs of rows each (94 KiB of LDS)
    n, k = 2048, 12288
    raw = synth.random_weight(dt, n, k, seed=dt + 40)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    for m in (3, 4):
        x = synth.random_activation(m, k, seed=50 + m)
        y = gpu.qmatmul(w, x, n, k)
        assert rel_l2(y, orc.matmul_dequant(dt, f16_round(x), raw, n, k)) <= 2e-5, m
    gpu.release(w)


@pytest.mark.parametrize("dt", [Q4_K, Q5_K])
def test_four_rows_several_weights_one_launch(gpu, dt):
    # gate + up against four rows: one launch of the packed form; every output equals the single call's bit for bit
    k, ns = 4096, [6144, 6100]
    raws = [synth.random_weight(dt, n, k, seed=n) for n in ns]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for n, raw in zip(ns, raws)]
    for m in (3, 4):
        x = synth.random_activation(m, k, seed=30 + m)
        ys = gpu.qmatmul_multi(ws, x, ns, k)
        for n, raw, w, y in zip(ns, raws, ws, ys):
            assert rel_l2(y, orc.matmul_dequant(dt, f16_round(x), raw, n, k)) <= 2e-5, (m, n)
            assert rel_l2(y, gpu.qmatmul(w, x, n, k)) <= 1e-5, (m, n)
    for w in ws:
        gpu.release(w)


@pytest.mark.parametrize("first", [Q4_K, Q5_K])
def test_two_rows_two_formats(gpu, first):
    # q, k (Q4_K or Q5_K) and v (Q6_K) against two activation rows: one launch of the two-format kernel
    k, ns, dts = 4096, [4096, 1024, 1000], (first, first, Q6_K)
    raws = [synth.random_weight(dt, n, k, seed=n + i) for i, (dt, n) in enumerate(zip(dts, ns))]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    x = synth.random_activation(2, k, seed=8, bf16=True)
    for x_dtype in (capi.ACT_F32, capi.ACT_BF16):
        ys = gpu.qmatmul_multi(ws, x, ns, k, x_dtype=x_dtype)
        for dt, n, raw, w, y in zip(dts, ns, raws, ws, ys):
            assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k)) <= 2e-5, (dt, n)
            # (the single call of a small weight takes another kernel: equal up to the order of the sums)
            assert rel_l2(y, gpu.qmatmul(w, x, n, k, x_dtype=x_dtype)) <= 1e-5, (dt, n)
    for w in ws:
        gpu.release(w)


def test_multi_weight_prefill_shares_the_preparation(gpu):
    # more than 32 rows with device pointers: the activations are prepared once per fragment order and every weight runs its
    # GEMM on them; the results are those of the single calls bit for bit (same kernels, same inputs)
    k, dts, ns = 1024, (Q4_K, Q6_K, Q8_0, Q8_0, Q5_K), [272, 64, 100, 48, 528]
    raws = [synth.random_weight(dt, n, k, seed=3 * i + n) for i, (dt, n) in enumerate(zip(dts, ns))]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    biases = [None if i == 2 else np.random.default_rng(i).standard_normal(n).astype(np.float32) for i, n in enumerate(ns)]
    for m in (33, 70, 200):
        x = synth.random_activation(m, k, seed=m, bf16=True)
        for x_dtype in (capi.ACT_F32, capi.ACT_BF16):
            ys = gpu.qmatmul_multi(ws, x, ns, k, x_dtype=x_dtype, biases=biases)
            for dt, n, raw, w, y, b in zip(dts, ns, raws, ws, ys, biases):
                assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k) + (0 if b is None else b)) <= 1e-3, (m, dt, n)
                assert np.array_equal(y, gpu.qmatmul(w, x, n, k, x_dtype=x_dtype, bias=b)), (m, dt, n)
    for w in ws:
        gpu.release(w)


def test_multi_weight_prefill_runs_of_one_format(gpu):
    # neighbouring weights of one K-quant format and shape (rows a multiple of 256) may go out as ONE launch of the prefill GEMM
    # whose n-blocks are dealt out to the weights; the rule only does that for weights that fill half the machine, so this test
    # also runs in a child process with every such run merged (test_prefill_merged_runs_forced).  Against the single calls
    # (other tiles, another order of the f32 sums where waves split k) and the oracle; biases, ragged m.
    k = 2048
    dts, ns = (Q5_K, Q5_K, Q5_K, Q6_K, Q6_K, Q6_K, Q6_K, Q4_K, Q4_K, Q8_0), [256, 256, 256, 512, 512, 512, 512, 256, 256, 64]
    raws = [synth.random_weight(dt, n, k, seed=5 * i + n) for i, (dt, n) in enumerate(zip(dts, ns))]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    biases = [None if i % 3 == 0 else np.random.default_rng(i).standard_normal(n).astype(np.float32) for i, n in enumerate(ns)]
    for m in (40, 130, 300):
        x = synth.random_activation(m, k, seed=m, bf16=True)
        ys = gpu.qmatmul_multi(ws, x, ns, k, x_dtype=capi.ACT_BF16, biases=biases)
        for i, (dt, n, raw, w, y, b) in enumerate(zip(dts, ns, raws, ws, ys, biases)):
            want = orc.matmul_dequant(dt, x, raw, n, k) + (0 if b is None else b)
            assert rel_l2(y, want) <= 1e-3, (m, i, dt)
            single = gpu.qmatmul(w, x, n, k, x_dtype=capi.ACT_BF16, bias=b)
            assert rel_l2(y, single) <= 2e-6, (m, i, dt, rel_l2(y, single))
    for w in ws:
        gpu.release(w)


def test_prefill_merged_runs_forced():
    import os
    import subprocess
    import sys

    env = dict(os.environ, TURQ_GEMM_MERGE="2")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "-k", "runs_of_one_format",
                          "-p", "no:cacheprovider", os.path.join(root, "tests", "test_gpu_qmatmul.py")],
                         cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-1000:]


def test_multi_weight_prefill_small_launches_side_by_side(gpu):
    # q / k / v of a prompt chunk: launches that leave half of the machine free run in groups of up to three, the first on
    # the context's stream, the others on further streams, between the shared preparation and the end of the call.  Same kernels, same inputs: bit-equal with the
    # single calls, eagerly (twice, the buffers reused) and in a captured graph replayed with other activations.
    L, ctx = gpu.L, gpu.ctx
    k, dts, ns = 1024, (Q4_K, Q4_K, Q6_K, Q5_K), [512, 128, 128, 80]
    raws = [synth.random_weight(dt, n, k, seed=7 * i + n) for i, (dt, n) in enumerate(zip(dts, ns))]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    biases = [np.random.default_rng(i).standard_normal(n).astype(np.float32) if i == 1 else None for i, n in enumerate(ns)]
    for m in (40, 130, 512, 40):
        x = synth.random_activation(m, k, seed=m, bf16=True)
        ys = gpu.qmatmul_multi(ws, x, ns, k, biases=biases)
        for dt, n, raw, w, y, b in zip(dts, ns, raws, ws, ys, biases):
            assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k) + (0 if b is None else b)) <= 1e-3, (m, dt, n)
            assert np.array_equal(y, gpu.qmatmul(w, x, n, k, bias=b)), (m, dt, n)

    def dev(nbytes):
        p = ctypes.c_void_p()
        capi.check(L.turq_dev_alloc(ctx, nbytes, ctypes.byref(p)), ctx)
        return p
    m = 96
    xd, yd = dev(m * k * 4), [dev(m * n * 4) for n in ns]
    warr = (ctypes.c_void_p * 4)(*[w.value for w in ws])
    yarr = (ctypes.c_void_p * 4)(*[p.value for p in yd])
    ldys = (ctypes.c_int64 * 4)(*ns)
    capi.check(L.turq_graph_begin(ctx), ctx)
    capi.check(L.turq_qmatmul_multi(ctx, 4, warr, xd, capi.ACT_F32, m, k, yarr, capi.ACT_F32, ldys, None, capi.MEM_DEVICE,
                                    capi.ALGO_AUTO), ctx)
    graph = ctypes.c_void_p()
    capi.check(L.turq_graph_end(ctx, ctypes.byref(graph)), ctx)
    for seed in (1, 2, 3):
        x = synth.random_activation(m, k, seed=seed, bf16=True)
        capi.check(L.turq_memcpy_h2d(ctx, xd, capi.ptr(x), x.nbytes), ctx)
        capi.check(L.turq_graph_launch(ctx, graph), ctx)
        capi.check(L.turq_sync(ctx), ctx)
        for w, n, p in zip(ws, ns, yd):
            y = np.zeros((m, n), np.float32)
            capi.check(L.turq_memcpy_d2h(ctx, capi.ptr(y), p, y.nbytes), ctx)
            assert np.array_equal(y, gpu.qmatmul(w, x, n, k)), (seed, n)   # eager work of the same context between the replays
    L.turq_graph_destroy(graph)
    for p in [xd] + yd:
        capi.check(L.turq_dev_free(ctx, p), ctx)
    for w in ws:
        gpu.release(w)


def test_multi_weight_falls_back_to_single_calls(gpu):
    # more than 32 rows, or host pointers: the same as the calls one after the other
    k, ns, dts = 512, [48, 80], (Q4_K, Q4_K)
    raws = [synth.random_weight(dt, n, k, seed=n) for dt, n in zip(dts, ns)]
    ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
    for m, mem in ((8, capi.MEM_DEVICE), (2, capi.MEM_HOST), (40, capi.MEM_DEVICE)):
        x = synth.random_activation(m, k, seed=m, bf16=True)      # exact in f16: only the kernels' own error is left
        ys = gpu.qmatmul_multi(ws, x, ns, k, mem=mem)
        for dt, n, raw, y in zip(dts, ns, raws, ys):
            # 40 rows take the prefill GEMM with its f16-folded scales, the others the exact skinny kernel
            assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k)) <= (1e-3 if m > 32 else 2e-5)
    # an argument a single call refuses is refused here too
    L, ctx = gpu.L, gpu.ctx
    warr = (ctypes.c_void_p * 2)(ws[0].value, None)
    yarr = (ctypes.c_void_p * 2)(None, None)
    ldys = (ctypes.c_int64 * 2)(*ns)
    assert L.turq_qmatmul_multi(ctx, 2, warr, None, capi.ACT_F32, 1, k, yarr, capi.ACT_F32, ldys, None, capi.MEM_DEVICE,
                                capi.ALGO_AUTO) == capi.ERR_INVALID
    assert L.turq_qmatmul_multi(ctx, 0, None, None, capi.ACT_F32, 1, k, None, capi.ACT_F32, None, None, capi.MEM_DEVICE,
                                capi.ALGO_AUTO) == capi.OK
    for w in ws:
        gpu.release(w)



# ---------------------------------------------------------------------------------------------
# every instantiation of the one-row kernel: the launch shape is normally derived from the matrix, so the
# environment overrides (read once per process) are applied to a child process running the tests above
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("row_tiles,in_flight", [(1, 1), (1, 2), (1, 3), (2, 1), (2, 2)])
def test_one_row_launch_shapes(row_tiles, in_flight):
    import os
    import subprocess
    import sys

    env = dict(os.environ, TURQ_ROW1_R=str(row_tiles), TURQ_ROW1_P=str(in_flight))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "-k", "test_one_row and not launch_shapes",
                          "-p", "no:cacheprovider", os.path.join(root, "tests", "test_gpu_qmatmul.py")],
                         cwd=root, env=env, capture_output=True, text=True, timeout=170)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-1000:]


# The kernel that keeps a column tile's activation fragments in registers (gemv_cs.hip) is picked for launches of several row
# tiles per compute unit, which the small matrices here never are: the batch tests run once more in child processes with each of
# its row-tile group sizes forced (every format, m = 2 .. 32, ragged shapes, strides, biases, all activation and output types).
@pytest.mark.parametrize("row_tiles", [2, 3, 6])
def test_rows_in_registers_kernel_shapes(row_tiles):
    import os
    import subprocess
    import sys

    env = dict(os.environ, TURQ_CS_RG=str(row_tiles))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    picked = ("test_mfma_gemv_tiled_layout or test_multi_weight_launch or test_activation_and_output_dtypes or test_bias_and_row_strides "
              "or test_q8_0_ragged_k or test_single_tile_shapes or test_mfma_more_rows_than_one_launch")
    out = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "-k", picked, "-p", "no:cacheprovider",
                          os.path.join(root, "tests", "test_gpu_qmatmul.py")], cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-1000:]


# 3 .. 32 rows on a k that splits evenly over the waves go through the form of that kernel that stages the activation rows
# through the LDS (no preparation launch, no scratch; more than 16 rows as two passes of 16 or, with several row tiles per
# workgroup and up to 4096 columns, in the four-wave form that takes both 16-row tiles per unpack).  A wave walks its column
# tiles in pairs: k = 512 is one pair for one wave, 1024 and 2048 one pair per wave, 4608 nine pairs for eight waves, 9728
# nineteen (waves with three and with two: the loop over pairs runs a different number of times per wave); n = 200 ends inside a row tile and, with several row tiles per workgroup, inside a workgroup.  One format
# and the two-format launches, every activation type, strides, biases, bf16 output; the rows of a batch are independent, so a
# batch of 32 equals four of 8.
@pytest.mark.parametrize("k", [512, 1024, 2048, 4608, 9728])
@pytest.mark.parametrize("dts", [(Q4_K,), (Q5_K,), (Q6_K,), (Q8_0,), (Q4_K, Q4_K, Q6_K), (Q5_K, Q6_K, Q6_K), (Q4_K, Q4_K, Q4_K, Q6_K)])
def test_staged_rows_kernel(dts, k):
    own = Gpu()
    try:
        ns = [200, 48, 33, 16][: len(dts)]
        raws = [synth.random_weight(dt, n, k, seed=11 * i + n + k) for i, (dt, n) in enumerate(zip(dts, ns))]
        ws = [own.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(dts, ns, raws)]
        biases = [None if i == 0 else np.random.default_rng(i).standard_normal(n).astype(np.float32) for i, n in enumerate(ns)]
        x16 = synth.random_activation(32, k, seed=k + len(dts), bf16=True)
        def scratch_bytes():
            live, retired, cap = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
            capi.check(own.L.turq_ctx_scratch_info(own.ctx, ctypes.byref(live), ctypes.byref(retired), ctypes.byref(cap)), own.ctx)
            return cap.value

        for m in (3, 5, 8, 9, 16, 17, 24, 32):
            x = x16[:m]
            for x_dtype in (capi.ACT_F32, capi.ACT_BF16, capi.ACT_F16):
                xv = f16_round(x) if x_dtype == capi.ACT_F16 else x
                ys = own.qmatmul_multi(ws, xv, ns, k, x_dtype=x_dtype, biases=biases)
                for dt, n, raw, y, b in zip(dts, ns, raws, ys, biases):
                    want = orc.matmul_dequant(dt, f16_round(xv), raw, n, k) + (0 if b is None else b)
                    assert rel_l2(y, want) <= 2e-5, (dt, n, m, x_dtype)
            # no fragments were prepared for any of these calls (more than 16 rows: on up to 4096 columns)
            if m <= 16 or k <= 4096:
                assert scratch_bytes() == 0, m
        # single calls: strides, bf16 store, and rows independent of the batch they are in
        for dt, n, raw, w, b in zip(dts, ns, raws, ws, biases):
            batch = x16 if k <= 4096 else x16[:16]       # (more rows on more columns take another kernel, with other sums)
            y = own.qmatmul(w, batch, n, k, bias=b, ldx=k + 8, ldy=n + 3)
            want = orc.matmul_dequant(dt, f16_round(batch), raw, n, k) + (0 if b is None else b)
            assert rel_l2(y, want) <= 2e-5
            for r0 in range(8, len(batch), 8):
                y8 = own.qmatmul(w, batch[r0:r0 + 8], n, k, bias=b)
                assert np.array_equal(y8, y[r0:r0 + 8])
            yb = own.qmatmul(w, x16[:7], n, k, x_dtype=capi.ACT_BF16, y_dtype=capi.ACT_BF16)
            assert rel_l2(yb, orc.matmul_dequant(dt, x16[:7], raw, n, k)) <= 4e-3      # bf16 store
        for w in ws:
            own.release(w)
    finally:
        own.close()


# ... and with each of its row-tile group sizes forced (the rule takes one row tile per workgroup for matrices this small)
@pytest.mark.parametrize("row_tiles", [2, 3, 6])
def test_staged_rows_kernel_group_sizes(row_tiles):
    import os
    import subprocess
    import sys

    env = dict(os.environ, TURQ_CS_RG=str(row_tiles))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "-k", "test_staged_rows_kernel and not group_sizes",
                          "-p", "no:cacheprovider", os.path.join(root, "tests", "test_gpu_qmatmul.py")],
                         cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-1000:]


# The prefill GEMM picks its tile (128 x 128, 128 x 192, the wide 128 x 256 with two-deep rings, or the low 64 x 128 for launches
# that would leave CUs idle) from the problem size; the small matrices of the tests above would never reach the wide one and
# always take the low one, so they run once more in child processes with each of the two forced and forbidden (the rule takes
# the wide tile for some of the full-size cases), and with the columns of every tile split over 2, 4 or 8 workgroups wherever
# that number divides the super-blocks (on the wide or the low tile), or never; and with the low tile's eight-wave form (two
# groups of waves on alternate super-blocks) forbidden, and forced on every low-tile launch with an even share of super-blocks.
@pytest.mark.parametrize("switch,value", [("TURQ_GEMM_WIDE", "1"), ("TURQ_GEMM_WIDE", "0"), ("TURQ_GEMM_LOW", "1"), ("TURQ_GEMM_LOW", "0"),
                                          ("TURQ_GEMM_SPLIT", "0"), ("TURQ_GEMM_SPLIT+TURQ_GEMM_SPLIT_FORM", "2+3"),
                                          ("TURQ_GEMM_SPLIT+TURQ_GEMM_SPLIT_FORM", "4+4"), ("TURQ_GEMM_SPLIT", "8"),
                                          ("TURQ_GEMM_KGROUPS", "1"), ("TURQ_GEMM_KGROUPS+TURQ_GEMM_LOW", "2+1"),
                                          ("TURQ_GEMM_KGROUPS+TURQ_GEMM_SPLIT+TURQ_GEMM_SPLIT_FORM", "2+2+4")])
def test_prefill_tile_shapes(switch, value):
    import os
    import subprocess
    import sys

    env = dict(os.environ, **dict(zip(switch.split("+"), value.split("+"))))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "gpu", "-k", "(prefill or more_rows) and not tile_shapes",
                          "-p", "no:cacheprovider", os.path.join(root, "tests", "test_gpu_qmatmul.py"),
                          os.path.join(root, "tests", "test_gpu_fullsize.py")],
                         cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-1000:]
