"""GPU parity of turq_embedding_lookup: rows of the dequantized table picked by token id, the lookup the reference does with
candle's Embedding on a table it dequantizes whole at load (src/models/layers/mod.rs:30-37).

Bar: bit-exact with the oracle's dequantize for f32 output (integer / byte work plus the separately rounded f32 operations of
to_float); bf16 / f16 outputs equal the oracle's values rounded once (round to nearest even).
"""
import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu
F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16 = 0, 1, 8, 12, 13, 14, 30
QUANT = [Q8_0, Q4_K, Q5_K, Q6_K]


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def lookup(gpu, w, ids, k, out_dtype=capi.ACT_F32, mem=capi.MEM_HOST, ldo=None):
    L, ctx = gpu.L, gpu.ctx
    ids = np.ascontiguousarray(ids, np.uint32)
    ldo = ldo or k
    ydt = {capi.ACT_F32: np.float32, capi.ACT_BF16: np.uint16, capi.ACT_F16: np.float16}[out_dtype]
    out = np.zeros((len(ids), ldo), ydt)
    if mem == capi.MEM_HOST:
        rc = L.turq_embedding_lookup(ctx, w, capi.ptr(ids), len(ids), capi.ptr(out), out_dtype, ldo, mem)
        capi.check(rc, ctx)
    else:
        idd, outd = ctypes.c_void_p(), ctypes.c_void_p()
        capi.check(L.turq_dev_alloc(ctx, max(ids.nbytes, 16), ctypes.byref(idd)), ctx)
        capi.check(L.turq_dev_alloc(ctx, max(out.nbytes, 16), ctypes.byref(outd)), ctx)
        capi.check(L.turq_memcpy_h2d(ctx, idd, capi.ptr(ids), ids.nbytes), ctx)
        capi.check(L.turq_memcpy_h2d(ctx, outd, capi.ptr(out), out.nbytes), ctx)
        capi.check(L.turq_embedding_lookup(ctx, w, idd, len(ids), outd, out_dtype, ldo, mem), ctx)
        capi.check(L.turq_memcpy_d2h(ctx, capi.ptr(out), outd, out.nbytes), ctx)
        capi.check(L.turq_dev_free(ctx, idd), ctx)
        capi.check(L.turq_dev_free(ctx, outd), ctx)
    return out


@pytest.mark.parametrize("dt", QUANT)
@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED])
@pytest.mark.parametrize("mem", [capi.MEM_HOST, capi.MEM_DEVICE])
def test_rows_equal_the_dequantized_table(gpu, dt, layout, mem):
    n, k = 1000 + 7, 512 + (32 if dt == Q8_0 else 0)       # ragged last row tile; Q8_0 rows that end inside a column tile
    raw = synth.random_weight(dt, n, k, seed=dt + layout)
    table = orc.dequantize(dt, raw).reshape(n, k)
    w = gpu.upload(dt, n, k, raw, layout)
    rng = np.random.default_rng(dt)
    ids = np.concatenate([[0, n - 1, n - 1, 16, 15], rng.integers(0, n, 40)]).astype(np.uint32)
    out = lookup(gpu, w, ids, k, mem=mem, ldo=k + 8)
    assert np.array_equal(out[:, :k].view(np.uint32), table[ids].view(np.uint32))
    assert np.all(out[:, k:] == 0)                          # the padding of the output rows is left alone
    gpu.release(w)


@pytest.mark.parametrize("dt", [F32, F16, BF16])
def test_dense_tables(gpu, dt):
    # token_embd of an F16 / BF16 / F32 GGUF file: the same call copies (and widens) the rows
    n, k = 300, 96
    vals = np.random.default_rng(dt).standard_normal((n, k)).astype(np.float32)
    if dt == F32:
        raw, table = vals.view(np.uint8), vals
    elif dt == F16:
        h = vals.astype(np.float16)
        raw, table = h.view(np.uint8), h.astype(np.float32)
    else:
        b = synth.to_bf16_bits(vals).reshape(n, k)
        raw, table = b.view(np.uint8), synth.from_bf16_bits(b).reshape(n, k)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_NATIVE)
    ids = np.array([5, 0, 299, 5], np.uint32)
    for mem in (capi.MEM_HOST, capi.MEM_DEVICE):
        assert np.array_equal(lookup(gpu, w, ids, k, mem=mem), table[ids])
    gpu.release(w)


@pytest.mark.parametrize("layout", [capi.LAYOUT_NATIVE, capi.LAYOUT_TILED])
def test_reduced_precision_outputs(gpu, layout):
    n, k = 64, 1024
    raw = synth.random_weight(Q6_K, n, k, seed=3)
    table = orc.dequantize(Q6_K, raw).reshape(n, k)
    w = gpu.upload(Q6_K, n, k, raw, layout)
    ids = np.arange(0, n, 3, dtype=np.uint32)
    ob = lookup(gpu, w, ids, k, out_dtype=capi.ACT_BF16, mem=capi.MEM_DEVICE)
    assert np.array_equal(ob, synth.to_bf16_bits(table[ids]).reshape(len(ids), k))
    oh = lookup(gpu, w, ids, k, out_dtype=capi.ACT_F16)
    assert np.array_equal(oh.view(np.uint16), table[ids].astype(np.float16).view(np.uint16))
    gpu.release(w)


def test_full_vocabulary_rows_and_batch_shape(gpu):
    # a prompt's worth of ids against a table with Qwen3's vocabulary size: every row equals the full dequantize
    n, k = 151936, 256
    raw = synth.random_weight(Q4_K, n, k, seed=9)
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_NATIVE)
    full = gpu.dequantize(w, n, k).reshape(n, k)
    ids = np.random.default_rng(1).integers(0, n, 2048).astype(np.uint32)
    out = lookup(gpu, w, ids, k, mem=capi.MEM_DEVICE)
    assert np.array_equal(out.view(np.uint32), full[ids].view(np.uint32))
    gpu.release(w)


def test_errors_empty_and_indices_outside_the_table(gpu):
    L, ctx = gpu.L, gpu.ctx
    n, k = 32, 256
    raw = synth.random_weight(Q4_K, n, k, seed=1)
    w = gpu.upload(Q4_K, n, k, raw, capi.LAYOUT_TILED)
    ids = np.array([1, 40, 2], np.uint32)
    out = np.full((3, k), 7.0, np.float32)
    # host indices are checked before anything runs
    assert L.turq_embedding_lookup(ctx, w, capi.ptr(ids), 3, capi.ptr(out), capi.ACT_F32, k, capi.MEM_HOST) == capi.ERR_INVALID
    assert "outside the table" in capi.last_error(ctx)
    assert np.all(out == 7.0)
    assert L.turq_embedding_lookup(ctx, w, capi.ptr(ids), 3, capi.ptr(out), capi.ACT_F32, k - 1, capi.MEM_HOST) == capi.ERR_SHAPE
    assert L.turq_embedding_lookup(ctx, w, capi.ptr(ids), -1, capi.ptr(out), capi.ACT_F32, k, capi.MEM_HOST) == capi.ERR_SHAPE
    assert L.turq_embedding_lookup(ctx, w, capi.ptr(ids), 3, capi.ptr(out), 9, k, capi.MEM_HOST) == capi.ERR_DTYPE
    assert L.turq_embedding_lookup(ctx, None, capi.ptr(ids), 3, capi.ptr(out), capi.ACT_F32, k, capi.MEM_HOST) == capi.ERR_INVALID
    assert L.turq_embedding_lookup(ctx, w, None, 3, capi.ptr(out), capi.ACT_F32, k, capi.MEM_HOST) == capi.ERR_INVALID
    assert L.turq_embedding_lookup(ctx, w, capi.ptr(ids), 0, capi.ptr(out), capi.ACT_F32, k, capi.MEM_HOST) == capi.OK
    assert np.all(out == 7.0)
    # device indices cannot be looked at by the call: the row of an index outside the table is NaN, the others are right
    got = lookup(gpu, w, ids, k, mem=capi.MEM_DEVICE)
    table = orc.dequantize(Q4_K, raw).reshape(n, k)
    assert np.array_equal(got[0], table[1]) and np.array_equal(got[2], table[2]) and np.all(np.isnan(got[1]))
    gpu.release(w)
