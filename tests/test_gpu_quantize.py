"""GPU parity: activation quantisation (Q8_0, Q8_K) is bit-exact with the oracle's from_float."""
import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def edge_rows(k, rng):
    rows = [rng.standard_normal(k).astype(np.float32) for _ in range(4)]
    z = np.zeros(k, np.float32)
    rows.append(z.copy())                                   # all-zero blocks
    a = rng.standard_normal(k).astype(np.float32)
    a[::7] = 0.0
    a[5] = -a[np.argmax(np.abs(a))] * 1.0                   # two elements share the largest magnitude, opposite sign
    rows.append(a)
    b = np.full(k, 0.5, np.float32)
    b[3::256] = 127.0                                       # products that land exactly on .5 (round half away)
    rows.append(b)
    c = np.full(k, -1.5, np.float32)
    c[1::32] = 127.0
    rows.append(c)
    d = rng.standard_normal(k).astype(np.float32) * np.float32(1e-30)   # tiny values: subnormal scales
    rows.append(d)
    e = rng.standard_normal(k).astype(np.float32) * np.float32(1e4)
    e[k - 1] = 7e4                                          # largest value last; f16 scale near overflow for Q8_0
    rows.append(e)
    return np.stack(rows)


@pytest.mark.parametrize("k", [256, 4096])
def test_quantize_q8_k_bit_exact(gpu, k):
    x = edge_rows(k, np.random.default_rng(k))
    got = gpu.quantize(x, "q8_k")
    want = np.concatenate([orc.quantize_q8_K(r) for r in x])
    assert np.array_equal(got, want)


@pytest.mark.parametrize("k", [32, 1024])
def test_quantize_q8_0_bit_exact(gpu, k):
    x = edge_rows(max(k, 256), np.random.default_rng(k + 1))[:, :k]
    got = gpu.quantize(np.ascontiguousarray(x), "q8_0")
    want = np.concatenate([orc.quantize_q8_0(r) for r in x])
    assert np.array_equal(got, want)


def test_quantize_rejects_ragged_k(gpu):
    from tur_amd import capi
    x = np.zeros((1, 100), np.float32)
    out = np.zeros(4096, np.uint8)
    assert gpu.L.turq_quantize_q8_k(gpu.ctx, capi.ptr(x), 1, 100, capi.ptr(out), capi.MEM_HOST) == capi.ERR_SHAPE
    assert gpu.L.turq_quantize_q8_0(gpu.ctx, capi.ptr(x), 1, 100, capi.ptr(out), capi.MEM_HOST) == capi.ERR_SHAPE
