"""turq_qmatmul_noalloc (the forward call that allocates nothing) against turq_qmatmul, through the C ABI.

Both run the same kernels, so the outputs must be bit-identical; the only difference is where the prepared activation
fragments live (a static device array instead of the context's growable buffer).  Two calls in a row, the second with a
smaller input, per launch kind: prepared fragments in the static array (17 .. 32 rows of a wide weight, a k that is not a
multiple of 512), the prefill GEMM (m > 32), and the kernels that use no scratch (one row; rows staged in the kernel).
One exception: prefill launches whose columns turq_qmatmul splits over several workgroups (few tiles: small or tall matrices
at prompt-chunk sizes) need a second scratch buffer for the partial tiles, which the call that allocates nothing does not
have; it runs the same kernel unsplit, i.e. the same products added up in another order, and is held to 2e-6 relative L2
against turq_qmatmul there (the bar of both against the oracle is 1e-3).
"""
from __future__ import annotations

import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu, rel_l2
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


def both(gpu, w, x, n, k, x_dtype, y_dtype):
    want = gpu.qmatmul_device(w, x, n, k, x_dtype=x_dtype, y_dtype=y_dtype)
    got = gpu.qmatmul_device(w, x, n, k, x_dtype=x_dtype, y_dtype=y_dtype, noalloc=True)
    return got, want


@pytest.mark.parametrize("dt,n,k,ms", [
    (capi.Q4_K, 4096, 4096, (32, 8)),       # up to 4096 columns: fragments made in the kernel from the rows themselves, no scratch
    (capi.Q6_K, 1024, 4096, (16, 3)),
    (capi.Q6_K, 4096, 12288, (32, 20)),     # 17 .. 32 rows of 12288 columns: fragments prepared in the static array, then fewer rows
    (capi.Q4_K, 2048, 4352, (24, 17)),      # k not a multiple of 512 (17 column tiles): prepared fragments again
    (capi.Q4_K, 1024, 4096, (512, 64)),     # the prefill GEMM, then a smaller chunk
    (capi.Q5_K, 512, 2048, (200, 33)),
    (capi.Q8_0, 3072, 1024, (48, 2)),
    (capi.Q4_K, 12288, 4096, (1, 1)),       # one row: no scratch at all
], ids=["q4k-staged", "q6k-staged", "q6k-frag-k12288", "q4k-frag-odd-k", "q4k-gemm", "q5k-gemm", "q8_0", "q4k-row1"])
def test_noalloc_equals_qmatmul_twice_in_a_row(gpu, dt, n, k, ms):
    raw = synth.random_weight(dt, n, k, seed=n + k)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    try:
        for i, m in enumerate(ms):
            x = synth.random_activation(m, k, seed=100 * i + m, bf16=True)
            got, want = both(gpu, w, x, n, k, capi.ACT_BF16, capi.ACT_F32)
            if m > 32 and not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
                assert (dt, n, k, m) in ((capi.Q4_K, 1024, 4096, 64), (capi.Q5_K, 512, 2048, 33)), "turq_qmatmul splits only these"
                assert rel_l2(got, want) <= 2e-6, (m, rel_l2(got, want))
            else:
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (m, "differs from turq_qmatmul")
            rows = np.arange(0, n, max(1, n * m // (1024 * 64)))
            sub = raw.reshape(n, -1)[rows].reshape(-1)
            assert rel_l2(got[:, rows], orc.matmul_dequant(dt, x, sub, len(rows), k)) <= 1e-3, m
    finally:
        gpu.release(w)


def test_noalloc_refuses_what_does_not_fit(gpu):
    L, ctx = gpu.L, gpu.ctx
    dt, n, k = capi.Q4_K, 64, 8192
    raw = synth.random_weight(dt, n, k, seed=3)
    w = gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED)
    try:
        m = 1024                              # 32 * 32 m-tiles x 32 column tiles x 17 KiB = 17.8 MB of fragments
        xd = gpu.dev_buffer(nbytes=m * k * 2)
        yd = gpu.dev_buffer(nbytes=m * n * 4)
        rc = L.turq_qmatmul_noalloc(ctx, w, xd, capi.ACT_BF16, m, k, yd, capi.ACT_F32, n, None)
        assert rc == capi.ERR_SHAPE
        assert "static scratch" in capi.last_error(ctx)
        # argument errors are turq_qmatmul's
        assert L.turq_qmatmul_noalloc(ctx, w, xd, capi.ACT_BF16, 4, k - 1, yd, capi.ACT_F32, n, None) == capi.ERR_SHAPE
        assert L.turq_qmatmul_noalloc(ctx, None, xd, capi.ACT_BF16, 4, k, yd, capi.ACT_F32, n, None) == capi.ERR_INVALID
        assert L.turq_qmatmul_noalloc(ctx, w, xd, capi.ACT_BF16, 0, k, yd, capi.ACT_F32, n, None) == capi.OK
        # and the ordinary entry point still takes the large call
        capi.check(L.turq_qmatmul(ctx, w, xd, capi.ACT_BF16, m, k, yd, capi.ACT_F32, n, None, capi.MEM_DEVICE, capi.ALGO_AUTO), ctx)
        capi.check(L.turq_sync(ctx), ctx)
        gpu.dev_free(xd)
        gpu.dev_free(yd)
    finally:
        gpu.release(w)


def test_noalloc_refuses_f32_rows_while_wide_activations_are_on():
    # wide activations need scratch of their own (the scaled f16 copy of the rows and a factor per row); the call that
    # allocates nothing says so instead of rounding f32 rows to f16 unscaled.  f16 rows need no scaling and still pass.
    g2 = Gpu()
    try:
        L, ctx = g2.L, g2.ctx
        dt, n, k, m = capi.Q4_K, 256, 1024, 8
        raw = synth.random_weight(dt, n, k, seed=4)
        w = g2.upload(dt, n, k, raw, capi.LAYOUT_TILED)
        x = synth.random_activation(m, k, seed=2, bf16=True)
        before = g2.qmatmul_device(w, x, n, k, x_dtype=capi.ACT_BF16, noalloc=True)
        capi.check(L.turq_ctx_set_wide_activations(ctx, 1), ctx)
        xd = g2.dev_buffer(nbytes=m * k * 4)
        yd = g2.dev_buffer(nbytes=m * n * 4)
        for xt in (capi.ACT_F32, capi.ACT_BF16):
            assert L.turq_qmatmul_noalloc(ctx, w, xd, xt, m, k, yd, capi.ACT_F32, n, None) == capi.ERR_INVALID
            assert "wide activations" in capi.last_error(ctx)
        x16 = x.astype(np.float16)
        y16 = g2.qmatmul_device(w, x16, n, k, x_dtype=capi.ACT_F16, noalloc=True)
        assert rel_l2(y16, orc.matmul_dequant(dt, x16.astype(np.float32), raw, n, k)) <= 2e-5
        capi.check(L.turq_ctx_set_wide_activations(ctx, 0), ctx)
        after = g2.qmatmul_device(w, x, n, k, x_dtype=capi.ACT_BF16, noalloc=True)
        assert np.array_equal(before.view(np.uint32), after.view(np.uint32))
        g2.dev_free(xd)
        g2.dev_free(yd)
        g2.release(w)
    finally:
        g2.close()


def test_noalloc_leaves_the_context_scratch_alone(gpu):
    # a fresh context: after calls through the no-allocation entry point its own fragment buffer is still unallocated
    g2 = Gpu()
    try:
        dt, n, k = capi.Q4_K, 256, 1024
        raw = synth.random_weight(dt, n, k, seed=9)
        w = g2.upload(dt, n, k, raw, capi.LAYOUT_TILED)
        x = synth.random_activation(8, k, seed=1, bf16=True)
        y = g2.qmatmul_device(w, x, n, k, x_dtype=capi.ACT_BF16, noalloc=True)
        assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, k)) <= 2e-5
        cap = ctypes.c_size_t(1)
        capi.check(g2.L.turq_ctx_scratch_info(g2.ctx, None, None, ctypes.byref(cap)), g2.ctx)
        assert cap.value == 0
        g2.release(w)
    finally:
        g2.close()
