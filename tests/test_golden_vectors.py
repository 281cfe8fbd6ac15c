"""Committed vectors (tests/golden/turq_vectors.npz, written by tests/golden/make_fixtures.py from the NumPy restatement):
the C oracle and the GPU kernels must reproduce them."""
from __future__ import annotations

import os

import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import rel_l2
from tur_amd import capi

VEC = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "turq_vectors.npz"))
DTYPES = {"q8_0": capi.Q8_0, "q4_k": capi.Q4_K, "q5_k": capi.Q5_K, "q6_k": capi.Q6_K}


@pytest.mark.parametrize("name", sorted(DTYPES))
def test_c_oracle_reproduces_the_vectors(name):
    dt = DTYPES[name]
    raw = VEC[f"{name}_raw"]
    n, k, m = (int(v) for v in VEC[f"{name}_shape"])
    assert np.array_equal(orc.dequantize(dt, raw).view(np.uint32), VEC[f"{name}_dequant_bits"])      # bit-exact
    x = VEC[f"{name}_x"]
    assert rel_l2(orc.matmul_dequant(dt, x, raw, n, k), VEC[f"{name}_dense"]) <= 1e-6
    # the restated CPU QMatMul: integer dot products are exact, only the f32 summation order may differ
    assert rel_l2(orc.qmatmul(dt, x, raw, n, k), VEC[f"{name}_cpu_qmatmul"]) <= 1e-5
    assert rel_l2(VEC[f"{name}_cpu_qmatmul"], VEC[f"{name}_dense"]) <= 1e-2


def test_c_oracle_quantizers_reproduce_the_vectors():
    x = VEC["quant_x"]
    assert np.array_equal(orc.quantize_q8_0(x).reshape(-1), VEC["quant_q8_0"].reshape(-1))
    assert np.array_equal(orc.quantize_q8_K(x).reshape(-1), VEC["quant_q8_k"].reshape(-1))


@pytest.fixture(scope="module")
def gpu():
    from tests.helpers import Gpu

    g = Gpu()
    yield g
    g.close()


@pytest.mark.gpu
@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED], ids=["native", "tiled"])
@pytest.mark.parametrize("name", sorted(DTYPES))
def test_gpu_reproduces_the_vectors(gpu, name, layout):
    dt = DTYPES[name]
    raw = VEC[f"{name}_raw"]
    n, k, m = (int(v) for v in VEC[f"{name}_shape"])
    w = gpu.upload(dt, n, k, raw, layout)
    assert np.array_equal(gpu.dequantize(w, n, k).view(np.uint32), VEC[f"{name}_dequant_bits"])      # bit-exact
    y = gpu.qmatmul(w, VEC[f"{name}_x"], n, k)
    gpu.release(w)
    assert rel_l2(y, VEC[f"{name}_dense"]) <= 1e-3
    assert rel_l2(y, VEC[f"{name}_cpu_qmatmul"]) <= 1e-2


@pytest.mark.gpu
def test_gpu_quantizers_reproduce_the_vectors(gpu):
    x = VEC["quant_x"]
    assert np.array_equal(gpu.quantize(x, "q8_0").reshape(-1), VEC["quant_q8_0"].reshape(-1))
    assert np.array_equal(gpu.quantize(x, "q8_k").reshape(-1), VEC["quant_q8_k"].reshape(-1))
