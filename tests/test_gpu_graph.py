"""A decode / prefill step captured into a HIP graph and replayed: every replay must give what the same calls give eagerly.

The step mixes the launch kinds a model step has: a q / k / v group of two formats (one launch at m = 1 and with prepared
fragments), a single call of a third format, and (m > 32) the prefill GEMM with its preparation kernel.  Between the replays
the program does its own eager work and synchronises, and the activations change in place, as they do between decode steps.
"""
from __future__ import annotations

import ctypes

import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import Gpu, rel_l2
from tur_amd import capi, synth

pytestmark = pytest.mark.gpu

Q8_0, Q4_K, Q6_K = capi.Q8_0, capi.Q4_K, capi.Q6_K


@pytest.fixture(scope="module")
def gpu():
    g = Gpu()
    yield g
    g.close()


class Step:
    """q / k / v (Q4_K, Q4_K, Q6_K) through turq_qmatmul_multi plus one Q8_0 matrix, everything in device memory."""

    def __init__(self, gpu, m, k=1024):
        self.gpu, self.m, self.k = gpu, m, k
        L, ctx = gpu.L, gpu.ctx
        self.dts = (Q4_K, Q4_K, Q6_K, Q8_0)
        self.ns = (80, 48, 33, 64)
        self.raws = [synth.random_weight(dt, n, k, seed=3 * i + n) for i, (dt, n) in enumerate(zip(self.dts, self.ns))]
        self.ws = [gpu.upload(dt, n, k, raw, capi.LAYOUT_TILED) for dt, n, raw in zip(self.dts, self.ns, self.raws)]
        self.bufs = []
        self.x = self._dev(m * k * 4)
        self.ys = [self._dev(m * n * 4) for n in self.ns]
        self.warr = (ctypes.c_void_p * 3)(*[w.value for w in self.ws[:3]])
        self.yarr = (ctypes.c_void_p * 3)(*[y.value for y in self.ys[:3]])
        self.ldys = (ctypes.c_int64 * 3)(*self.ns[:3])

    def _dev(self, nbytes):
        p = ctypes.c_void_p()
        capi.check(self.gpu.L.turq_dev_alloc(self.gpu.ctx, nbytes, ctypes.byref(p)), self.gpu.ctx)
        self.bufs.append(p)
        return p

    def close(self):
        for b in self.bufs:
            capi.check(self.gpu.L.turq_dev_free(self.gpu.ctx, b), self.gpu.ctx)
        for w in self.ws:
            self.gpu.release(w)

    def set_x(self, x):
        x = np.ascontiguousarray(x, np.float32)
        capi.check(self.gpu.L.turq_memcpy_h2d(self.gpu.ctx, self.x, capi.ptr(x), x.nbytes), self.gpu.ctx)

    def clear_outputs(self):
        for y, n in zip(self.ys, self.ns):
            z = np.full(self.m * n, np.nan, np.float32)
            capi.check(self.gpu.L.turq_memcpy_h2d(self.gpu.ctx, y, capi.ptr(z), z.nbytes), self.gpu.ctx)

    def outputs(self):
        capi.check(self.gpu.L.turq_sync(self.gpu.ctx), self.gpu.ctx)
        outs = []
        for y, n in zip(self.ys, self.ns):
            o = np.empty((self.m, n), np.float32)
            capi.check(self.gpu.L.turq_memcpy_d2h(self.gpu.ctx, capi.ptr(o), y, o.nbytes), self.gpu.ctx)
            outs.append(o)
        return outs

    def calls(self):
        L, ctx, m, k = self.gpu.L, self.gpu.ctx, self.m, self.k
        capi.check(L.turq_qmatmul_multi(ctx, 3, self.warr, self.x, capi.ACT_F32, m, k, self.yarr, capi.ACT_F32, self.ldys, None,
                                        capi.MEM_DEVICE, capi.ALGO_AUTO), ctx)
        capi.check(L.turq_qmatmul(ctx, self.ws[3], self.x, capi.ACT_F32, m, k, self.ys[3], capi.ACT_F32, self.ns[3], None,
                                  capi.MEM_DEVICE, capi.ALGO_AUTO), ctx)


# (64 rows of 8192 columns: prefill launches whose tiles are split over several workgroups - their counters in device memory
# must be back at zero after every replay, with no memset node in the graph)
@pytest.mark.parametrize("m,k", [(1, 1024), (8, 1024), (64, 1024), (64, 8192)])
def test_graph_replays_equal_the_eager_calls(gpu, m, k):
    L, ctx = gpu.L, gpu.ctx
    st = Step(gpu, m, k=k)
    other = Step(gpu, 3, k=512)          # the program's own eager work between replays
    other.set_x(synth.random_activation(3, 512, seed=99))
    try:
        st.set_x(synth.random_activation(m, st.k, seed=1))
        st.calls()                        # scratch buffers reach their final size outside the capture
        capi.check(L.turq_sync(ctx), ctx)
        capi.check(L.turq_graph_begin(ctx), ctx)
        st.calls()
        g = ctypes.c_void_p()
        capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
        assert g.value
        for rep in range(4):
            x = synth.random_activation(m, st.k, seed=10 + rep)
            st.set_x(x)
            st.clear_outputs()
            st.calls()
            want = st.outputs()
            for dt, n, raw, y in zip(st.dts, st.ns, st.raws, want):
                assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, st.k)) <= 1e-3, (rep, dt)
            other.calls()                 # eager work of another shape: the shared scratch buffers are rewritten
            other.outputs()
            st.clear_outputs()
            capi.check(L.turq_graph_launch(ctx, g), ctx)
            got = st.outputs()
            for dt, y, w in zip(st.dts, got, want):
                assert np.array_equal(y, w), (rep, dt)
        L.turq_graph_destroy(g)
    finally:
        st.close()
        other.close()


def test_graph_misuse_is_an_error_not_a_crash(gpu):
    L, ctx = gpu.L, gpu.ctx
    g = ctypes.c_void_p()
    assert L.turq_graph_end(ctx, ctypes.byref(g)) == capi.ERR_INVALID          # no capture running
    assert L.turq_graph_launch(ctx, None) == capi.ERR_INVALID
    capi.check(L.turq_graph_begin(ctx), ctx)
    assert L.turq_graph_begin(ctx) == capi.ERR_INVALID                         # already capturing
    capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)                    # an empty graph is still a graph
    capi.check(L.turq_graph_launch(ctx, g), ctx)
    capi.check(L.turq_sync(ctx), ctx)
    L.turq_graph_destroy(g)
    L.turq_graph_destroy(None)


def scratch_info(gpu):
    live, retired, cap = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    capi.check(gpu.L.turq_ctx_scratch_info(gpu.ctx, ctypes.byref(live), ctypes.byref(retired), ctypes.byref(cap)), gpu.ctx)
    return live.value, retired.value, cap.value


def test_scratch_that_grows_under_a_live_graph_is_kept_for_it():
    # a graph captured at m = 40 refers to the fragment buffer by address; a later, larger eager call (m = 64 on a wider
    # matrix) makes that buffer grow.  The old buffer must stay allocated while the graph is alive (the replay below then
    # reads and writes valid memory and gives the eager result again), and is released once no graph is alive.
    gpu = Gpu()                           # a context of its own: the bookkeeping starts from zero
    L, ctx = gpu.L, gpu.ctx
    st = Step(gpu, 40)                    # more than 32 rows: the kernels read fragments prepared in the context's scratch
    big = Step(gpu, 64, k=4096)
    try:
        x = synth.random_activation(40, st.k, seed=5)
        st.set_x(x)
        st.calls()
        want = st.outputs()
        assert scratch_info(gpu)[:2] == (0, 0)
        cap0 = scratch_info(gpu)[2]
        capi.check(L.turq_graph_begin(ctx), ctx)
        st.calls()
        g = ctypes.c_void_p()
        capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
        assert scratch_info(gpu)[:2] == (1, 0)
        big.set_x(synth.random_activation(64, big.k, seed=6))
        big.calls()                       # needs more scratch than the capture left behind
        big.outputs()
        live, retired, cap1 = scratch_info(gpu)
        assert cap1 > cap0 and (live, retired) == (1, 1)
        for _ in range(2):
            st.clear_outputs()
            capi.check(L.turq_graph_launch(ctx, g), ctx)
            got = st.outputs()
            for y, w in zip(got, want):
                assert np.array_equal(y, w)
        L.turq_graph_destroy(g)
        assert scratch_info(gpu)[0] == 0
        huge = Step(gpu, 128, k=8192)      # the next growth finds no live graph and lets the retired buffer go
        try:
            huge.set_x(synth.random_activation(128, huge.k, seed=7))
            huge.calls()
            huge.outputs()
            assert scratch_info(gpu)[:2] == (0, 0)
        finally:
            huge.close()
    finally:
        st.close()
        big.close()
        gpu.close()


def test_a_call_that_fails_inside_a_capture_ends_it():
    gpu = Gpu()
    L, ctx = gpu.L, gpu.ctx
    st = Step(gpu, 40)
    try:
        x = synth.random_activation(40, st.k, seed=8)
        st.set_x(x)
        capi.check(L.turq_graph_begin(ctx), ctx)
        # first use of the fragment buffer inside a capture: it would have to be allocated, which a capture does not allow
        rc = L.turq_qmatmul_multi(ctx, 3, st.warr, st.x, capi.ACT_F32, 40, st.k, st.yarr, capi.ACT_F32, st.ldys, None,
                                  capi.MEM_DEVICE, capi.ALGO_AUTO)
        assert rc == capi.ERR_INVALID
        assert "capture" in capi.last_error(ctx)
        g = ctypes.c_void_p()
        assert L.turq_graph_end(ctx, ctypes.byref(g)) == capi.ERR_INVALID      # the capture is gone
        assert not g.value
        st.calls()                                                             # stream and context are usable again
        want = st.outputs()
        for dt, n, raw, y in zip(st.dts, st.ns, st.raws, want):
            assert rel_l2(y, orc.matmul_dequant(dt, x, raw, n, st.k)) <= 1e-3
        capi.check(L.turq_graph_begin(ctx), ctx)                               # and so is capturing
        st.calls()
        capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
        st.clear_outputs()
        capi.check(L.turq_graph_launch(ctx, g), ctx)
        for y, w in zip(st.outputs(), want):
            assert np.array_equal(y, w)
        L.turq_graph_destroy(g)
    finally:
        st.close()
        gpu.close()


def test_read_yardstick_is_timed_like_a_kernel(gpu):
    """turq_read_yardstick: a launch that only reads; with kernel timing on it counts as one timed launch, and it refuses
    pointers the kernel's 16-byte loads could not take"""
    L, ctx = gpu.L, gpu.ctx
    nbytes = 8 << 20
    buf = gpu.dev_buffer(np.zeros(nbytes // 4, np.float32))
    capi.check(L.turq_read_yardstick(ctx, buf, nbytes), ctx)
    capi.check(L.turq_profile_begin(ctx), ctx)
    for _ in range(3):
        capi.check(L.turq_read_yardstick(ctx, buf, nbytes), ctx)
    n, ms = ctypes.c_int64(), ctypes.c_double()
    capi.check(L.turq_profile_end(ctx, ctypes.byref(n), ctypes.byref(ms)), ctx)
    assert n.value == 3 and 0.0 < ms.value < 50.0
    assert L.turq_read_yardstick(ctx, ctypes.c_void_p(buf.value + 4), 4096) == capi.ERR_INVALID
    assert L.turq_read_yardstick(ctx, None, 4096) == capi.ERR_INVALID
    assert L.turq_read_yardstick(ctx, buf, 100) == capi.OK      # less than one 4 KiB chunk: nothing to launch
    capi.check(L.turq_sync(ctx), ctx)
    gpu.dev_free(buf)


def test_weight_prefetch_changes_no_result_eager_or_captured():
    """turq_weight_prefetch is a hint: a read-only pass on a stream of the context's own.  The calls around it give the same
    bits with and without it, eagerly and as a parallel branch of a captured graph (replayed with eager work in between), and a
    capture that holds such a branch ends cleanly."""
    gpu = Gpu()
    L, ctx = gpu.L, gpu.ctx
    st = Step(gpu, 1, k=2048)
    other = Step(gpu, 3, k=512)
    other.set_x(synth.random_activation(3, 512, seed=98))

    def hinted():
        capi.check(L.turq_weight_prefetch(ctx, st.ws[3]), ctx)     # the weight of the second call, next to the first
        capi.check(L.turq_qmatmul_multi(ctx, 3, st.warr, st.x, capi.ACT_F32, st.m, st.k, st.yarr, capi.ACT_F32, st.ldys, None,
                                        capi.MEM_DEVICE, capi.ALGO_AUTO), ctx)
        for w in st.ws[:3]:                                         # the next step's first weights, next to the second
            capi.check(L.turq_weight_prefetch(ctx, w), ctx)
        capi.check(L.turq_qmatmul(ctx, st.ws[3], st.x, capi.ACT_F32, st.m, st.k, st.ys[3], capi.ACT_F32, st.ns[3], None,
                                  capi.MEM_DEVICE, capi.ALGO_AUTO), ctx)

    try:
        assert L.turq_weight_prefetch(ctx, None) == capi.ERR_INVALID
        st.set_x(synth.random_activation(1, st.k, seed=21))
        st.calls()
        want = st.outputs()
        st.clear_outputs()
        hinted()
        for y, w in zip(st.outputs(), want):
            assert np.array_equal(y, w)
        capi.check(L.turq_graph_begin(ctx), ctx)
        hinted()
        g = ctypes.c_void_p()
        capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
        for rep in range(3):
            st.set_x(synth.random_activation(1, st.k, seed=30 + rep))
            st.clear_outputs()
            st.calls()
            want = st.outputs()
            other.calls()
            other.outputs()
            st.clear_outputs()
            capi.check(L.turq_graph_launch(ctx, g), ctx)
            for y, w in zip(st.outputs(), want):
                assert np.array_equal(y, w), rep
        L.turq_graph_destroy(g)
    finally:
        st.close()
        other.close()
        gpu.close()
