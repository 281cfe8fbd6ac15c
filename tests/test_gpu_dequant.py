"""GPU parity: turq_dequantize is bit-exact with the oracle's to_float for every format, in both
HBM layouts, including hand-built edge blocks (subnormal / zero / largest f16 scales, extreme
quants and scales)."""
import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def edge_blocks(dt, rng):
    """blocks whose scale fields walk through the awkward f16 values and extreme integer fields"""
    f16_vals = np.array([0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF, 0x3C00, 0x0010, 0x8001, 0x3555, 0x6400],
                        np.uint16)
    nb = len(f16_vals) * 2
    blk = synth.random_blocks(dt, nb, rng)
    doff = {Q8_0: 0, Q4_K: 0, Q5_K: 0, Q6_K: 208}[dt]
    for i in range(nb):
        blk[i, doff:doff + 2] = np.array([f16_vals[i % len(f16_vals)]], np.uint16).view(np.uint8)
        if dt in (Q4_K, Q5_K):
            blk[i, 2:4] = np.array([f16_vals[(i * 5 + 3) % len(f16_vals)]], np.uint16).view(np.uint8)
    if dt in (Q4_K, Q5_K):
        blk[0, 4:16] = 0xFF            # all scales and mins 63
        blk[1, 4:16] = 0x00
        blk[2, 16:] = 0xFF             # all quants (and Q5_K high bits) at maximum
        blk[3, 16:] = 0x00
    elif dt == Q6_K:
        blk[0, 192:208] = 0x80         # scales -128
        blk[1, 192:208] = 0x7F         # scales 127
        blk[2, 0:192] = 0xFF
        blk[3, 0:192] = 0x00
    else:
        blk[0, 2:] = 0x80              # -128
        blk[1, 2:] = 0x7F
    return blk


@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED])
@pytest.mark.parametrize("dt", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_dequantize_bit_exact_random(gpu, dt, layout):
    n, k = 70, 1280
    raw = synth.random_weight(dt, n, k, seed=dt + 100 * layout)
    w = gpu.upload(dt, n, k, raw, layout)
    got = gpu.dequantize(w, n, k)
    gpu.release(w)
    want = orc.dequantize(dt, raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED])
@pytest.mark.parametrize("dt", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_dequantize_bit_exact_edge_blocks(gpu, dt, layout):
    rng = np.random.default_rng(7)
    blk = edge_blocks(dt, rng)
    be = synth.BLOCK_ELEMS[dt]
    n, k = 2, blk.shape[0] // 2 * be
    raw = blk.reshape(-1)
    w = gpu.upload(dt, n, k, raw, layout)
    got = gpu.dequantize(w, n, k)
    gpu.release(w)
    want = orc.dequantize(dt, raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dt", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_export_round_trips_through_hbm(gpu, dt):
    n, k = 37, 768
    raw = synth.random_weight(dt, n, k, seed=dt)
    for layout in (capi.LAYOUT_NATIVE, capi.LAYOUT_TILED):
        w = gpu.upload(dt, n, k, raw, layout)
        back = gpu.export(w, raw.size)
        gpu.release(w)
        assert np.array_equal(raw, back)


@pytest.mark.parametrize("dt,npdt", [(0, "<f4"), (1, "<f2")])
def test_dequantize_dense_tensors(gpu, dt, npdt):
    # norm weights and biases arrive as F32 / F16 GGUF tensors and take the same dequantize call
    v = np.random.default_rng(1).standard_normal(4096).astype(npdt)
    w = gpu.upload(dt, 1, 4096, v.view(np.uint8), capi.LAYOUT_NATIVE)
    got = gpu.dequantize(w, 1, 4096)
    gpu.release(w)
    assert np.array_equal(got, v.astype(np.float32))


def test_dequantize_bf16_tensor(gpu):
    x = np.random.default_rng(2).standard_normal(512).astype(np.float32)
    bits = synth.to_bf16_bits(x)
    w = gpu.upload(30, 1, 512, bits.view(np.uint8), capi.LAYOUT_NATIVE)
    got = gpu.dequantize(w, 1, 512)
    gpu.release(w)
    assert np.array_equal(got, synth.from_bf16_bits(bits))


def test_dequantize_full_size_row_block(gpu):
    # Qwen3-8B gate_proj geometry, a 256-row slab of it: checksum of the whole slab against the oracle
    n, k = 256, 4096
    raw = synth.random_weight(Q4_K, n, k, seed=11)
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_TILED)
    got = gpu.dequantize(w, n, k)
    gpu.release(w)
    want = orc.dequantize(Q4_K, raw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
