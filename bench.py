#!/usr/bin/env python3
"""Benchmark of the GGUF quantized-linear hot path on one MI355X.

Default workload (the configuration the headline metric is quoted on): Q4_K decode GEMV at the
Qwen3-8B MLP shapes - gate_proj and up_proj [12288 x 4096], down_proj [4096 x 12288] - at m = 1.
One "step" is one decode pass over the MLPs of `--layers` decoder layers (default 36, the depth of
Qwen3-8B): 3 * layers quantized matmuls, each on its OWN copy of the weights in HBM, so a step
streams layers * 84.9 MB (3.06 GB by default) and nothing is served from the 256 MB Infinity
Cache.  Inputs are resident in HBM when the clock starts.  Matrices that take the same input (gate
and up; q, k and v) are issued through turq_qmatmul_multi, as the reference calls them back to back
on one tensor: for up to four activation rows that is one kernel launch per run of equal formats
(`--single-calls` issues one turq_qmatmul per matrix instead).  The step is captured once into a HIP
graph and replayed (one graph launch per step).

Prints ONE JSON line.  `value` is whole-step algorithmic bytes (weights + activations + outputs)
per second (TFLOP/s for the prefill workload).  `roofline` prices the matmul kernels alone:
algorithmic bytes (or flops) of the step over the sum of the kernel durations, i.e. per average
launch, measured with HIP events stamped with every kernel's own begin and end in a second, untimed
pass of the same steps.  `cpu_baseline` times the oracle's restatement of candle's CPU QMatMul
(quantise activations to Q8_K, integer dot products) on the host cores on one layer's matmuls.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from tur_amd import capi, synth  # noqa: E402

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, vendor figure
MFMA_F16_PEAK_TFLOPS = 2500.0   # dense f16 / bf16 MFMA, vendor figure
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.md")


def load_traffic():
    """HBM bytes per launch of the timed kernels (average over the launches of a step), measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE and scaled by the same counters on a copy kernel of known size: the rows of the table in
    profiles/hbm_traffic_per_launch.md, which names the commands and the commit they ran on.  Keyed by (workload, m,
    activations, calls); a leg that has no row reports null."""
    table = {}
    try:
        with open(TRAFFIC_TABLE) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 5 and cells[1].isdigit() and cells[4].replace(" ", "").isdigit():
                    table[(cells[0].strip("`"), int(cells[1]), cells[2], cells[3])] = int(cells[4].replace(" ", ""))
    except OSError:
        pass
    return table


TRAFFIC = load_traffic()

WORKLOADS = {
    # name: (description, [(label, ggml dtype, n, k), ...] per layer)
    "q4k_mlp_8b": ("Q4_K GEMV, Qwen3-8B MLP (gate/up 12288x4096, down 4096x12288)", synth.CONFIGS["q4k_mlp_8b"]),
    "q4km_layer_8b": ("Q4_K_M mixed decoder layer, Qwen3-8B (Q6_K v/down, Q4_K q/k/o/gate/up)", synth.CONFIGS["q4km_layer_8b"]),
    "q8_0_gate_0p6b": ("Q8_0 GEMV, Qwen3-0.6B gate_proj 3072x1024", synth.CONFIGS["q8_0_gate_0p6b"]),
    "lm_head_q6k_8b": ("LM head Q6_K 151936x4096", synth.CONFIGS["lm_head_q6k_8b"]),
    "lm_head_q5k_8b": ("LM head Q5_K 151936x4096", synth.CONFIGS["lm_head_q5k_8b"]),
    "q4k_prefill_up_8b": ("chunked-prefill GEMM, Qwen3-8B up_proj Q4_K 12288x4096 (use --m 512 or 2048, --act bf16 --out bf16)",
                          synth.CONFIGS["q4k_prefill_up_8b"]),
}
OUT = {"f32": (capi.ACT_F32, 4), "bf16": (capi.ACT_BF16, 2)}
ACT = {"f32": (capi.ACT_F32, 4, np.float32), "bf16": (capi.ACT_BF16, 2, np.uint16)}


# projections that the reference applies to one and the same tensor (src/models/qwen3.rs:272-274 and :161-167); o_proj and
# down_proj have inputs of their own
SHARED_INPUT = ({"q", "k", "v"}, {"gate", "up"})


def shares_input(a, b):
    return any(a in g and b in g for g in SHARED_INPUT)


def algorithmic_bytes(dt, n, k, m, xbytes, ybytes):
    return synth.weight_nbytes(dt, n, k) + m * k * xbytes + m * n * ybytes


class Bench:
    def __init__(self, args):
        self.args = args
        self.L = capi.lib()
        self.ctx = ctypes.c_void_p()
        capi.check(self.L.turq_ctx_create(0, ctypes.byref(self.ctx)))
        name = ctypes.create_string_buffer(128)
        cus = ctypes.c_int()
        capi.check(self.L.turq_ctx_device_info(self.ctx, name, 128, ctypes.byref(cus)), self.ctx)
        self.device = name.value.decode()
        self.cus = cus.value
        self.desc, self.mats = WORKLOADS[args.workload]
        if getattr(args, "rows", None):
            self.mats = [(label, dt, args.rows, k) for label, dt, _, k in self.mats]
            self.desc += f" [weight rows overridden: {args.rows}]"
        self.xt, self.xbytes, self.xnp = ACT[args.act]
        self.yt, self.ybytes = OUT[args.out]
        self.weights = []      # [layer][matrix] -> handle
        self.host_raw = {}     # label -> raw bytes of the first layer (CPU baseline, checks)
        self.calls = []        # (weight, x_dev, y_dev, n, k)
        self.x_dev, self.y_dev = {}, []
        self._setup()
        self.set_m(args.m)

    def dev_alloc(self, nbytes):
        p = ctypes.c_void_p()
        capi.check(self.L.turq_dev_alloc(self.ctx, nbytes, ctypes.byref(p)), self.ctx)
        return p

    def _setup(self):
        L, ctx = self.L, self.ctx
        layers = self.args.layers
        per_layer = sum(synth.weight_nbytes(dt, n, k) for _, dt, n, k in self.mats)
        if per_layer * layers > 200e9:
            raise SystemExit("workload does not fit: lower --layers")
        # one set of seeded weights; every layer gets its own device copy (distinct HBM addresses)
        raws = []
        for i, (label, dt, n, k) in enumerate(self.mats):
            raw = synth.random_weight(dt, n, k, seed=1000 + i)
            raws.append(raw)
            self.host_raw[label] = raw
        for _ in range(layers):
            row = []
            for (label, dt, n, k), raw in zip(self.mats, raws):
                w = ctypes.c_void_p()
                capi.check(L.turq_weight_upload(ctx, dt, n, k, capi.ptr(raw), raw.size, capi.LAYOUT_TILED, ctypes.byref(w)), ctx)
                row.append(w)
            self.weights.append(row)

    def set_m(self, m):
        """(re)allocate the activations and outputs for m rows: one resident input per distinct k, one output per matrix"""
        L, ctx, layers = self.L, self.ctx, self.args.layers
        for p in list(self.x_dev.values()) + list(self.y_dev):
            capi.check(L.turq_dev_free(ctx, p), ctx)
        if getattr(self, "glue", None):
            for key in ("xres", "xn", "nw", "tmp"):
                capi.check(L.turq_dev_free(ctx, self.glue[key]), ctx)
            self.glue = None
        self.m = m
        self.calls = []
        self.x_host = {}
        self.x_dev = {}
        for _, _, n, k in self.mats:
            if k not in self.x_dev:
                x = synth.random_activation(self.m, k, seed=k, bf16=(self.args.act == "bf16"))
                if self.use_mlp():
                    # the synthetic weights give products of a few hundred at unit activations and act(gate) * up would leave
                    # the f16 range that down_proj rounds its input to: a power of two keeps the bf16 values exact
                    x = x * np.float32(2.0 ** -7)
                self.x_host[k] = x
                send = synth.to_bf16_bits(x).reshape(self.m, k) if self.args.act == "bf16" else x
                p = self.dev_alloc(send.nbytes)
                capi.check(L.turq_memcpy_h2d(ctx, p, capi.ptr(send), send.nbytes), ctx)
                self.x_dev[k] = p
        self.y_dev = [self.dev_alloc(self.m * n * self.ybytes) for _, _, n, _ in self.mats]
        for layer in self.weights:
            for (label, dt, n, k), w, y in zip(self.mats, layer, self.y_dev):
                self.calls.append((w, self.x_dev[k], y, n, k))
        # neighbouring matrices that take the same input (gate/up, q/k/v) go through turq_qmatmul_multi, as the
        # reference calls them back to back on one tensor (src/models/qwen3.rs:161-167, 272-274)
        self.groups = []       # (count, weight array, x, y array, ldy array, k)
        labels = [mt[0] for mt in self.mats]
        for layer in self.weights:
            i = 0
            while i < len(self.mats):
                if self.use_mlp() and labels[i:i + 3] == ["gate", "up", "down"]:
                    # the whole MLP through turq_mlp (src/models/qwen3.rs:161-167): x -> down_proj's output
                    warr = (ctypes.c_void_p * 3)(*[w.value for w in layer[i:i + 3]])
                    yarr = (ctypes.c_void_p * 1)(self.y_dev[i + 2].value)
                    ldys = (ctypes.c_int64 * 1)(self.mats[i + 2][2])
                    self.groups.append((3, warr, self.x_dev[self.mats[i][3]], yarr, ldys, self.mats[i][3], "mlp"))
                    i += 3
                    continue
                j = i + 1
                while j < len(self.mats) and self.mats[j][3] == self.mats[i][3] and shares_input(self.mats[i][0], self.mats[j][0]):
                    j += 1
                cnt = j - i
                warr = (ctypes.c_void_p * cnt)(*[w.value for w in layer[i:j]])
                yarr = (ctypes.c_void_p * cnt)(*[y.value for y in self.y_dev[i:j]])
                ldys = (ctypes.c_int64 * cnt)(*[mt[2] for mt in self.mats[i:j]])
                fused = bool(getattr(self.args, "gate_up", False)) and [mt[0] for mt in self.mats[i:j]] == ["gate", "up"]
                self.groups.append((cnt, warr, self.x_dev[self.mats[i][3]], yarr, ldys, self.mats[i][3], fused))
                i = j
        self.step_bytes = layers * sum(algorithmic_bytes(dt, n, k, self.m, self.xbytes, self.ybytes) for _, dt, n, k in self.mats)
        if getattr(self.args, "gate_up", False):
            # turq_qmatmul_gate_up reads the shared activations once and writes one output for the pair
            self.step_bytes -= layers * sum(self.m * (n * self.ybytes + k * self.xbytes) for lb, _, n, k in self.mats if lb == "up")
        if self.use_mlp():
            # one input, one output; the f32 intermediate (m * 12288 floats written and read back) is not counted
            self.step_bytes -= layers * sum(self.m * (n * self.ybytes + (k * self.xbytes if lb == "up" else 0))
                                            for lb, _, n, k in self.mats if lb in ("gate", "up"))
            self.step_bytes -= layers * sum(self.m * k * self.xbytes for lb, _, n, k in self.mats if lb == "down")
        self.step_flops = layers * sum(2 * self.m * n * k for _, _, n, k in self.mats)

    def calls_label(self):
        a = self.args
        if getattr(a, "glue", None):
            return ("turq_norm_qmatmul_multi + turq_qmatmul (accumulate) + turq_norm_mlp (accumulate)" if a.glue == "fused"
                    else "turq_rms_norm + turq_qmatmul_multi + turq_qmatmul + turq_rms_norm + turq_mlp")
        return ("turq_qmatmul" if a.single_calls else "turq_mlp + turq_qmatmul_multi" if self.use_mlp()
                else "turq_qmatmul_gate_up + turq_qmatmul_multi" if a.gate_up else "turq_qmatmul_multi")

    def reconfigure(self, m, act=None, out=None, mlp=None, glue=None):
        """another leg on the same resident weights: activation / output types, turq_mlp per layer or not, m rows"""
        if act is not None:
            self.args.act = act
            self.xt, self.xbytes, self.xnp = ACT[act]
        if out is not None:
            self.args.out = out
            self.yt, self.ybytes = OUT[out]
        if mlp is not None:
            self.args.mlp = mlp
        self.args.glue = glue
        self.set_m(m)

    def use_mlp(self):
        """gate / up / down as one turq_mlp call per layer (--mlp)"""
        labels = [mt[0] for mt in self.mats]
        has = any(labels[i:i + 3] == ["gate", "up", "down"] for i in range(len(labels)))
        return has and bool(getattr(self.args, "mlp", False)) and not self.args.single_calls and not self.args.gate_up

    def setup_glue(self):
        """buffers of the decoder layer's linear path with its glue (--glue): the residual stream, the attention block's output
        (random: attention itself is not part of this path), the normalised rows of the separate form, the norm weight"""
        if getattr(self, "glue", None) and self.glue["m"] == self.m:
            return
        L, ctx, m = self.L, self.ctx, self.m
        labels = [mt[0] for mt in self.mats]
        if labels != ["q", "k", "v", "o", "gate", "up", "down"] or self.args.act != self.args.out:
            raise SystemExit("--glue needs the decoder-layer workload (q4km_layer_8b) and --act equal to --out")
        k = self.mats[0][3]
        g = {"m": m, "k": k}
        x0 = synth.random_activation(m, k, seed=7, bf16=(self.args.act == "bf16"))
        g["x0"] = synth.to_bf16_bits(x0).reshape(m, k) if self.args.act == "bf16" else x0
        g["x0_f32"] = x0
        g["xres"] = self.dev_alloc(g["x0"].nbytes)
        g["xn"] = self.dev_alloc(g["x0"].nbytes)
        g["attn"] = self.x_dev[k]
        # a norm weight of 2^-7: the synthetic weights give products of a few hundred at unit activations, and
        # act(gate) * up of such rows would leave the f16 range that down_proj rounds its input to
        nw = np.full(k, 2.0 ** -7, np.float32)
        g["nw_host"] = nw
        g["nw"] = self.dev_alloc(nw.nbytes)
        capi.check(L.turq_memcpy_h2d(ctx, g["nw"], capi.ptr(nw), nw.nbytes), ctx)
        g["tmp"] = self.dev_alloc(m * k * self.ybytes)
        self.glue = g
        self.reset_glue()

    def reset_glue(self):
        g = self.glue
        capi.check(self.L.turq_memcpy_h2d(self.ctx, g["xres"], capi.ptr(g["x0"]), g["x0"].nbytes), self.ctx)

    def step_glue(self, layers=None):
        """the reference's decoder layer without its attention block (src/models/qwen3.rs:633-640): ln1 -> q / k / v, o_proj added
        to the residual stream, ln2 -> MLP added to it; --glue fused: three calls per layer, --glue separate: the norms as calls
        of their own and the projections into buffers (the two additions are then the engine's own launches, not made here)"""
        L, ctx, m, xt, yt, g = self.L, self.ctx, self.m, self.xt, self.yt, self.glue
        k, eps, acc = g["k"], 1e-6, capi.OUT_ACCUMULATE
        fused = self.args.glue == "fused"
        for li, layer in enumerate(self.weights if layers is None else self.weights[:layers]):
            wq, wk, wv, wo, wg, wu, wd = layer
            warr = (ctypes.c_void_p * 3)(wq.value, wk.value, wv.value)
            yarr = (ctypes.c_void_p * 3)(*[y.value for y in self.y_dev[:3]])
            ldys = (ctypes.c_int64 * 3)(*[mt[2] for mt in self.mats[:3]])
            if fused:
                rc = L.turq_norm_qmatmul_multi(ctx, 3, warr, g["xres"], xt, m, k, g["nw"], eps, yarr, yt, ldys, None, capi.MEM_DEVICE)
                rc = rc or L.turq_qmatmul(ctx, wo, g["attn"], xt, m, k, g["xres"], yt | acc, k, None, capi.MEM_DEVICE, capi.ALGO_AUTO)
                rc = rc or L.turq_norm_mlp(ctx, wg, wu, wd, g["xres"], xt, m, k, g["nw"], eps, g["xres"], yt | acc, k, None, None, None,
                                           capi.ACTFN_SILU, capi.MEM_DEVICE)
            else:
                rc = L.turq_rms_norm(ctx, g["xres"], xt, m, k, k, g["nw"], eps, g["xn"], xt, k, capi.MEM_DEVICE)
                rc = rc or L.turq_qmatmul_multi(ctx, 3, warr, g["xn"], xt, m, k, yarr, yt, ldys, None, capi.MEM_DEVICE, capi.ALGO_AUTO)
                rc = rc or L.turq_qmatmul(ctx, wo, g["attn"], xt, m, k, g["tmp"], yt, k, None, capi.MEM_DEVICE, capi.ALGO_AUTO)
                rc = rc or L.turq_rms_norm(ctx, g["xres"], xt, m, k, k, g["nw"], eps, g["xn"], xt, k, capi.MEM_DEVICE)
                rc = rc or L.turq_mlp(ctx, wg, wu, wd, g["xn"], xt, m, k, g["tmp"], yt, k, None, None, None, capi.ACTFN_SILU, capi.MEM_DEVICE)
            if rc:
                capi.check(rc, ctx)

    def verify_glue(self):
        """first layer of the fused form against the oracle: the q projection of the normalised rows, and the residual stream
        after the layer (first rows only; the chain needs every column)"""
        from oracle import capi as orc
        from oracle import oracle_np as onp
        g, m = self.glue, self.m
        keep = min(m, 8)
        self.reset_glue()
        saved = self.args.glue
        self.args.glue = "fused"
        self.step_glue(layers=1)
        self.args.glue = saved
        self.sync()
        k = g["k"]
        x = g["x0_f32"][:keep].astype(np.float64)
        xn = (x / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-6) * g["nw_host"]).astype(np.float32)
        by = {mt[0]: mt for mt in self.mats}

        def fetch(ptr, n):
            a = np.empty((m, n), np.float32 if self.yt == capi.ACT_F32 else np.uint16)
            capi.check(self.L.turq_memcpy_d2h(self.ctx, capi.ptr(a), ptr, a.nbytes), self.ctx)
            return (a if self.yt == capi.ACT_F32 else synth.from_bf16_bits(a).reshape(m, n))[:keep]

        def rnd(a):
            return a if self.yt == capi.ACT_F32 else synth.from_bf16_bits(synth.to_bf16_bits(np.asarray(a, np.float32))).reshape(np.shape(a))

        _, dq, nq, _ = by["q"]
        want_q = orc.matmul_dequant(dq, xn, self.host_raw["q"], nq, k)
        rel_q = float(np.linalg.norm(fetch(self.y_dev[0], nq) - rnd(want_q)) / np.linalg.norm(want_q))
        attn = self.x_host[k][:keep]
        x1 = g["x0_f32"][:keep] + orc.matmul_dequant(by["o"][1], attn, self.host_raw["o"], k, k)
        x1 = rnd(x1).astype(np.float64)
        xn2 = (x1 / np.sqrt((x1 * x1).mean(axis=1, keepdims=True) + 1e-6) * g["nw_host"]).astype(np.float32)
        h = onp.silu_mul(orc.matmul_dequant(by["gate"][1], xn2, self.host_raw["gate"], by["gate"][2], k),
                         orc.matmul_dequant(by["up"][1], xn2, self.host_raw["up"], by["up"][2], k))
        want = x1 + orc.matmul_dequant(by["down"][1], h, self.host_raw["down"], by["down"][2], by["down"][3])
        rel_x = float(np.linalg.norm(fetch(g["xres"], k) - rnd(want)) / np.linalg.norm(want))
        bar = 1e-3 if self.yt == capi.ACT_F32 else 3e-3
        if rel_q > bar or rel_x > 2 * bar:
            raise SystemExit(f"bench: --glue differs from the oracle (q {rel_q:.3e}, residual stream {rel_x:.3e}; bar {bar})")
        self.reset_glue()
        return max(rel_q, rel_x)

    def step_eager(self):
        if getattr(self.args, "glue", None):
            return self.step_glue()
        L, ctx, m, xt = self.L, self.ctx, self.m, self.xt
        ahead = int(getattr(self.args, "prefetch", 0) or 0)
        if not self.args.single_calls:
            for gi, (cnt, warr, x, yarr, ldys, k, fused) in enumerate(self.groups):
                if ahead:
                    # the weights of the call `ahead` calls further on (the next step's first ones after the last call): read
                    # next to this call's launch, in the reference's order of calls
                    ncnt, nwarr = self.groups[(gi + ahead) % len(self.groups)][:2]
                    for t in range(ncnt):
                        rc = L.turq_weight_prefetch(ctx, nwarr[t])
                        if rc:
                            capi.check(rc, ctx)
                if fused == "mlp":
                    rc = L.turq_mlp(ctx, warr[0], warr[1], warr[2], x, xt, m, k, yarr[0], self.yt, ldys[0], None, None, None,
                                    capi.ACTFN_SILU, capi.MEM_DEVICE)
                    if rc:
                        capi.check(rc, ctx)
                    continue
                if fused:
                    rc = L.turq_qmatmul_gate_up(ctx, warr[0], warr[1], x, xt, m, k, yarr[0], self.yt, ldys[0], None, None,
                                                capi.ACTFN_SILU, capi.MEM_DEVICE)
                    if rc:
                        capi.check(rc, ctx)
                    continue
                rc = L.turq_qmatmul_multi(ctx, cnt, warr, x, xt, m, k, yarr, self.yt, ldys, None, capi.MEM_DEVICE, capi.ALGO_AUTO)
                if rc:
                    capi.check(rc, ctx)
            return
        for w, x, y, n, k in self.calls:
            rc = L.turq_qmatmul(ctx, w, x, xt, m, k, y, self.yt, n, None, capi.MEM_DEVICE, capi.ALGO_AUTO)
            if rc:
                capi.check(rc, ctx)

    def sync(self):
        capi.check(self.L.turq_sync(self.ctx), self.ctx)

    def verify(self):
        """first layer's outputs against the oracle (small m only; it is a sanity gate, not the parity suite)"""
        from oracle import capi as orc
        self.step_eager()
        self.sync()
        worst = 0.0
        fused = bool(getattr(self.args, "gate_up", False)) and not self.args.single_calls
        mlp = self.use_mlp()
        by_label = {mt[0]: mt for mt in self.mats}
        for (label, dt, n, k), y in zip(self.mats, self.y_dev):
            if fused and label == "up":
                continue      # its product went into the gate's output
            if mlp and label in ("gate", "up"):
                continue      # only down_proj's output leaves the call
            got = np.empty((self.m, n), np.float32 if self.yt == capi.ACT_F32 else np.uint16)
            capi.check(self.L.turq_memcpy_d2h(self.ctx, capi.ptr(got), y, got.nbytes), self.ctx)
            if self.yt != capi.ACT_F32:
                got = synth.from_bf16_bits(got).reshape(self.m, n)
            rows = np.arange(0, n, max(1, (n * self.m) // (4096 * 16)))      # bounded CPU time at prefill sizes
            got = got[:, rows]
            sub = self.host_raw[label].reshape(n, -1)[rows].reshape(-1)
            if mlp and label == "down":
                from oracle import oracle_np as onp
                _, gdt, gn, gk = by_label["gate"]
                keep = min(self.m, 16)      # the chain needs every column of the intermediate: bounded by checking the first rows only
                got = got[:keep]
                xg = self.x_host[gk][:keep].astype(np.float16).astype(np.float32)
                h = onp.silu_mul(orc.matmul_dequant(gdt, xg, self.host_raw["gate"], gn, gk), orc.matmul_dequant(gdt, xg, self.host_raw["up"], gn, gk))
                want = orc.matmul_dequant(dt, h, sub, len(rows), k)
            else:
                want = orc.matmul_dequant(dt, self.x_host[k], sub, len(rows), k)
            if fused and label == "gate":
                from oracle import oracle_np as onp
                sub_up = self.host_raw["up"].reshape(n, -1)[rows].reshape(-1)
                want = onp.silu_mul(want, orc.matmul_dequant(dt, self.x_host[k], sub_up, len(rows), k))
            if self.yt != capi.ACT_F32:
                # a bf16 store alone costs about 1.6e-3: the oracle's result is rounded the same way, so that what is left is
                # the kernel's own error (and the elements it tips into the neighbouring bf16 value)
                want = synth.from_bf16_bits(synth.to_bf16_bits(np.asarray(want, np.float32))).reshape(np.shape(want))
            rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
            worst = max(worst, rel)
        # (the MLP is two matmuls in a row, each inside its own bar)
        bar = (1e-3 if self.yt == capi.ACT_F32 else 2e-3) * (2 if mlp and self.m > 32 else 1)
        if worst > bar:
            raise SystemExit(f"bench: output differs from the oracle (rel-L2 {worst:.3e} > {bar})")
        return worst

    def measure(self, steps, warmup):
        """verify against the oracle, time `steps` steps (whole step), then time the matmul kernels alone"""
        a = self.args
        L, ctx = self.L, self.ctx
        if getattr(a, "glue", None):
            self.setup_glue()
            rel = self.verify_glue()
            self.step_eager()      # (scratch buffers reach their size outside the capture)
            self.sync()
            self.reset_glue()
        else:
            rel = self.verify()
        graph = None
        if not a.eager:
            capi.check(L.turq_graph_begin(ctx), ctx)
            self.step_eager()
            g = ctypes.c_void_p()
            capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
            graph = g
        one = (lambda: capi.check(L.turq_graph_launch(ctx, graph), ctx)) if graph else self.step_eager
        for _ in range(warmup):
            one()
        self.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            one()
        self.sync()
        dt_s = time.perf_counter() - t0
        ms_per_step = dt_s / steps * 1e3
        gbps = self.step_bytes / (dt_s / steps) / 1e9

        # dominant kernel alone: event pairs around every matmul kernel launch, same steps, untimed pass
        n_launch = ctypes.c_int64()
        tot_ms = ctypes.c_double()
        # (the timed steps were graph replays: one pass from the host first, which also counts the launches of a step)
        capi.check(L.turq_profile_begin(ctx), ctx)
        self.step_eager()
        capi.check(L.turq_profile_end(ctx, ctypes.byref(n_launch), ctypes.byref(tot_ms)), ctx)
        per_step = max(1, n_launch.value)
        # at least 100 launches behind the average (an LM head step is two launches), at most 60 steps
        prof_steps = min(60, max(1, min(steps, 10), -(-100 // per_step)))
        # three passes, the median of their averages: launches made one by one from the host leave the GPU idle in between,
        # and a pass's average moves by a few per cent with it (the graph-replayed step above does not)
        passes = []
        for _ in range(3):
            capi.check(L.turq_profile_begin(ctx), ctx)
            for _ in range(prof_steps):
                self.step_eager()
            capi.check(L.turq_profile_end(ctx, ctypes.byref(n_launch), ctypes.byref(tot_ms)), ctx)
            passes.append(tot_ms.value / max(1, n_launch.value) * 1e3)
        avg_us = sorted(passes)[1]
        # all timed launches are the matmul kernel (one per matrix, or one per group of matrices with a common input)
        bytes_per_launch = self.step_bytes * prof_steps / max(1, n_launch.value)
        achieved = bytes_per_launch / (avg_us * 1e-6) / 1e9
        if graph:
            L.turq_graph_destroy(graph)
        traffic = TRAFFIC.get((a.workload, self.m, a.act, self.calls_label()))
        if self.m > 32:
            flops_per_launch = self.step_flops * prof_steps / max(1, n_launch.value)
            tfl = flops_per_launch / (avg_us * 1e-6) / 1e12
            roofline = {
                "bound": "mfma", "achieved": round(tfl, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tfl / MFMA_F16_PEAK_TFLOPS, 4), "traffic": traffic,
                "kernel": "gemm_kq_kernel", "avg_launch_us": round(avg_us, 3), "launches_timed": n_launch.value,
                "flops_per_launch": int(flops_per_launch),
            }
            value, unit = self.step_flops / (dt_s / steps) / 1e12, "TFLOP/s"
        else:
            roofline = {
                "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                "kernel": "gemv_row1_kernel" if self.m == 1 else "gemv_cs_staged_kernel / gemv_multi_frag_kernel" if self.m > 2 else "gemv_row1_kernel / gemv_multi_kernel", "avg_launch_us": round(avg_us, 3), "launches_timed": n_launch.value,
                "algorithmic_bytes_per_launch": int(bytes_per_launch),
            }
            value, unit = gbps, "GB/s"
        return {"value": value, "unit": unit, "ms_per_step": ms_per_step, "gbps": gbps, "roofline": roofline, "rel": rel}

    def run(self):
        a = self.args
        r = self.measure(a.steps, a.warmup)
        if self.m > 32:
            what = "Q4_K, Qwen3-8B up_proj" if a.workload == "q4k_prefill_up_8b" else a.workload
            metric = f"quantized prefill GEMM TFLOP/s ({what})"
        else:
            metric = "quantized GEMV HBM GB/s (Q4_K/Q6_K, Qwen3-8B shapes)"
        out = {
            "metric": metric,
            "value": round(r["value"], 1), "unit": r["unit"], "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "ms_per_step": round(r["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": f"{a.workload}: {self.desc}", "m": self.m, "layers": a.layers,
                       "activations": a.act, "outputs": a.out, "launch": "eager" if a.eager else "hip-graph",
                       "calls": self.calls_label(),
                       "step_bytes": int(self.step_bytes), "device": self.device, "compute_units": self.cus,
                       "max_rel_l2_vs_oracle": float(f"{r['rel']:.3e}")},
            "whole_step_gbps": round(r["gbps"], 1), "pct_of_hbm_peak": round(100 * r["gbps"] / HBM_PEAK_GBPS, 2),
            "roofline": r["roofline"],
            "cpu_baseline": self.cpu_baseline() if not a.no_cpu else None,
        }
        return out

    def calibrate_copy(self, nelem=64 * 1024 * 1024):
        L, ctx = self.L, self.ctx
        src = np.zeros(nelem, np.float32)
        w = ctypes.c_void_p()
        capi.check(L.turq_weight_upload(ctx, capi.F32, 1, nelem, capi.ptr(src), src.nbytes, capi.LAYOUT_NATIVE, ctypes.byref(w)), ctx)
        dst = self.dev_alloc(src.nbytes)
        for _ in range(3):
            capi.check(L.turq_dequantize(ctx, w, dst, capi.MEM_DEVICE), ctx)
        self.sync()
        capi.check(L.turq_dev_free(ctx, dst), ctx)
        capi.check(L.turq_weight_release(w))

    def cpu_baseline(self):
        """restated candle CPU QMatMul (quantise activations, integer vec_dot) on one layer's matmuls"""
        from oracle import capi as orc
        cores = min(os.cpu_count() or 1, 16)
        layer_bytes = sum(algorithmic_bytes(dt, n, k, self.m, 4, 4) for _, dt, n, k in self.mats)
        budget_s = 12.0
        reps, t_used = 0, 0.0
        while t_used < budget_s:
            t0 = time.perf_counter()
            for label, dt, n, k in self.mats:
                orc.qmatmul(dt, self.x_host[k], self.host_raw[label], n, k, nthreads=cores)
            t_used += time.perf_counter() - t0
            reps += 1
        if self.m > 32:
            layer_flops = sum(2 * self.m * n * k for _, _, n, k in self.mats)
            return {"value": round(layer_flops * reps / t_used / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                    "sample": f"{reps} passes over one layer's matmuls ({len(self.mats)} calls, m={self.m}) in {t_used:.1f} s; "
                              "restated candle CPU QMatMul (not candle itself), gcc -O3 scalar vec_dot, OpenMP over output columns"}
        return {"value": round(layer_bytes * reps / t_used / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"{reps} passes over one layer's matmuls ({len(self.mats)} calls, m={self.m}) in {t_used:.1f} s; "
                          "restated candle CPU QMatMul (not candle itself), gcc -O3 scalar vec_dot, OpenMP over output columns"}

    def close(self):
        for layer in self.weights:
            for w in layer:
                self.L.turq_weight_release(w)
        self.L.turq_ctx_destroy(self.ctx)


def run_embedding(args):
    """Side measurement (not the headline): turq_embedding_lookup of --m token ids on a token_embd-sized table
    [151936, 4096] Q6_K in the native layout, ids and output in HBM; a step is one call, replayed from a HIP graph."""
    from oracle import capi as orc
    L = capi.lib()
    ctx = ctypes.c_void_p()
    capi.check(L.turq_ctx_create(0, ctypes.byref(ctx)))
    n, k, dt, count = 151936, 4096, synth.Q6_K, args.m
    raw = synth.random_weight(dt, n, k, seed=77)
    w = ctypes.c_void_p()
    capi.check(L.turq_weight_upload(ctx, dt, n, k, capi.ptr(raw), raw.size, capi.LAYOUT_NATIVE, ctypes.byref(w)), ctx)
    ids = np.random.default_rng(5).integers(0, n, count).astype(np.uint32)
    idd, outd = ctypes.c_void_p(), ctypes.c_void_p()
    capi.check(L.turq_dev_alloc(ctx, max(ids.nbytes, 16), ctypes.byref(idd)), ctx)
    capi.check(L.turq_dev_alloc(ctx, count * k * 4, ctypes.byref(outd)), ctx)
    capi.check(L.turq_memcpy_h2d(ctx, idd, capi.ptr(ids), ids.nbytes), ctx)
    call = lambda: capi.check(L.turq_embedding_lookup(ctx, w, idd, count, outd, capi.ACT_F32, k, capi.MEM_DEVICE), ctx)
    call()
    got = np.empty((count, k), np.float32)
    capi.check(L.turq_memcpy_d2h(ctx, capi.ptr(got), outd, got.nbytes), ctx)
    rows = raw.reshape(n, -1)[ids[:64]].reshape(-1)
    if not np.array_equal(got[:64].view(np.uint32), orc.dequantize(dt, rows).reshape(-1, k).view(np.uint32)):
        raise SystemExit("bench: embedding rows differ from the oracle's dequantize")
    reps = 64      # calls per graph: one graph launch costs the host about 20 us, more than a small lookup takes
    capi.check(L.turq_graph_begin(ctx), ctx)
    for _ in range(reps):
        call()
    g = ctypes.c_void_p()
    capi.check(L.turq_graph_end(ctx, ctypes.byref(g)), ctx)
    one = lambda: capi.check(L.turq_graph_launch(ctx, g), ctx)
    for _ in range(args.warmup):
        one()
    capi.check(L.turq_sync(ctx), ctx)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one()
    capi.check(L.turq_sync(ctx), ctx)
    dt_s = (time.perf_counter() - t0) / (args.steps * reps)
    nbytes = count * (k // 256 * 210 + 4 + 4 * k)      # blocks of the rows + the ids read, f32 rows written
    print(json.dumps({"metric": "embedding lookup HBM GB/s (token_embd Q6_K 151936x4096, rows dequantized on gather)",
                      "value": round(nbytes / dt_s / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                      "ms_per_step": round(dt_s * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                      "dtype": "f32", "data": "synthetic",
                      "config": {"workload": "token_embd_q6k_8b", "ids": count, "layout": "native", "launch": "hip-graph of 64 calls", "step": "one call",
                                 "bytes_per_step": nbytes, "checked": "first 64 rows bit-equal to the oracle"}}))
    L.turq_graph_destroy(g)
    capi.check(L.turq_weight_release(w))
    L.turq_ctx_destroy(ctx)


def default_layers(per_layer):
    # enough distinct weight copies that a step streams well over the 256 MB Infinity Cache
    return max(36 if per_layer < 200e6 else 2, -(-768_000_000 // per_layer))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="q4k_mlp_8b", choices=sorted(WORKLOADS))
    ap.add_argument("--m", type=int, default=1, help="activation rows (decode batch)")
    ap.add_argument("--layers", type=int, default=None, help="distinct weight copies streamed per step")
    ap.add_argument("--rows", type=int, default=None,
                    help="side measurement: every matrix of the workload with this many weight rows instead of its own (how a "
                         "prefill launch's time depends on the number of workgroups: q4k_prefill_up_8b with 1536 .. 24576 rows)")
    ap.add_argument("--act", default="f32", choices=sorted(ACT))
    ap.add_argument("--out", default="f32", choices=sorted(OUT), help="output element type")
    ap.add_argument("--eager", action="store_true", help="launch every call from the host instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="default workload only: leave out the prefill GEMM, mixed-layer and LM-head legs of the JSON line")
    ap.add_argument("--prefetch", type=int, default=0,
                    help="turq_weight_prefetch on the weights of the call this many calls ahead, issued in front of every call")
    ap.add_argument("--single-calls", action="store_true",
                    help="one turq_qmatmul per matrix instead of turq_qmatmul_multi per group of matrices with a common input")
    ap.add_argument("--mlp", action="store_true",
                    help="the whole MLP through turq_mlp (down_proj takes act(gate) * up; the activations are scaled by 2^-7 so that the "
                         "synthetic intermediate stays in the f16 range) instead of gate / up and down on independent activations")
    ap.add_argument("--glue", choices=["fused", "separate"], default=None,
                    help="decoder-layer workload: the layer's linear path WITH its norms and residual additions (no attention): 'fused' = "
                         "turq_norm_qmatmul_multi, turq_qmatmul and turq_norm_mlp with TURQ_OUT_ACCUMULATE (three calls per layer), "
                         "'separate' = turq_rms_norm calls and plain projections (five calls, the two additions left to the engine)")
    ap.add_argument("--gate-up", action="store_true",
                    help="gate_proj / up_proj through turq_qmatmul_gate_up (SiLU and the product applied in the call, one output)")
    ap.add_argument("--embedding", action="store_true",
                    help="side measurement: turq_embedding_lookup of --m ids on a [151936, 4096] Q6_K table instead of a matmul workload")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before the workload, run a plain copy kernel of known size (dequantize of an F32 tensor: 256 MiB "
                         "read + 256 MiB written) three times, as the yardstick for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.embedding:
        return run_embedding(args)
    if args.layers is None:
        per_layer = sum(synth.weight_nbytes(dt, args.rows or n, k) for _, dt, n, k in WORKLOADS[args.workload][1])
        args.layers = default_layers(per_layer)
    headline = not args.rows and all(getattr(args, f) == ap.get_default(f) for f in ("workload", "m", "act", "out")) and not (
        args.eager or args.single_calls or args.gate_up or args.mlp or args.calibrate_copy or args.glue or args.prefetch)
    b = Bench(args)
    try:
        if args.calibrate_copy:
            b.calibrate_copy()
        out = b.run()
        if headline and not args.no_extra:
            out.update(other_halves(args, b))
    finally:
        b.close()
    print(json.dumps(out), flush=True)


def leg(b, ms, act, outdt, steps, warmup, mlp=False, glue=None):
    """one leg of the metric on the weights Bench b holds: a row per m, measured like the headline"""
    rows = []
    for m in ms:
        b.reconfigure(m, act, outdt, mlp, glue)
        r = b.measure(steps, warmup)
        rf = r["roofline"]
        rows.append({"m": m, "value": round(r["value"], 1), "unit": r["unit"], "ms_per_step": round(r["ms_per_step"], 4),
                     "bound": rf["bound"], "kernel_achieved": rf["achieved"], "frac": rf["frac"], "traffic": rf["traffic"],
                     "avg_launch_us": rf["avg_launch_us"], "launches_timed": rf["launches_timed"],
                     "max_rel_l2_vs_oracle": float(f"{r['rel']:.3e}")})
    wl = b.args.workload
    return {"workload": f"{wl}: {WORKLOADS[wl][0]}", "layers": b.args.layers, "activations": act, "outputs": outdt,
            "calls": b.calls_label(), "peaks": {"hbm": HBM_PEAK_GBPS, "mfma": MFMA_F16_PEAK_TFLOPS},
            "oracle_check": ("max_rel_l2_vs_oracle: f32 outputs against the f32 matmul on the dequantized weights, bar 1e-3" if outdt == "f32" else
                             "max_rel_l2_vs_oracle: bf16 outputs against that matmul's result rounded to bf16 the same way, bar 2e-3 (a bf16 "
                             "store alone is 1.6e-3 away from the f32 value; what is left are the elements the kernel's own error, 3e-4, tips "
                             "into the neighbouring bf16 value; the GPU tests hold the f32 result to 1e-3 and the bf16 store to bit equality "
                             "with the rounded f32 result)"),
            "rows": rows}


def bench_for(base, workload):
    args = argparse.Namespace(**vars(base))
    args.workload, args.mlp = workload, False
    per_layer = sum(synth.weight_nbytes(dt, n, k) for _, dt, n, k in WORKLOADS[workload][1])
    args.layers = default_layers(per_layer)
    return Bench(args)


def read_floor():
    """What a launch that only READS the bytes of a decode launch takes (turq_read_yardstick: one 16-wave workgroup per compute
    unit, the shape of the decode kernels), timed like the kernels.  The sizes are those of the launches of the two decode
    workloads; each launch reads a region of its own of a 2 GiB buffer, so nothing is served from a cache."""
    L = capi.lib()
    ctx = ctypes.c_void_p()
    capi.check(L.turq_ctx_create(0, ctypes.byref(ctx)))
    total = 2 << 30
    buf = ctypes.c_void_p()
    rows = []
    try:
        capi.check(L.turq_dev_alloc(ctx, total, ctypes.byref(buf)), ctx)
        w = ctypes.c_void_p()   # dequantizing a 64 MiB F32 tensor into every part of the buffer touches (and so maps) all of it
        one = np.zeros(16 << 20, np.float32)
        capi.check(L.turq_weight_upload(ctx, capi.F32, 1, one.size, capi.ptr(one), one.nbytes, capi.LAYOUT_NATIVE, ctypes.byref(w)), ctx)
        for part in range(total // one.nbytes):
            capi.check(L.turq_dequantize(ctx, w, ctypes.c_void_p(buf.value + part * one.nbytes), capi.MEM_DEVICE), ctx)
        capi.check(L.turq_sync(ctx), ctx)
        capi.check(L.turq_weight_release(w))
        sizes = {"o_proj Q4_K 4096x4096": synth.weight_nbytes(synth.Q4_K, 4096, 4096),
                 "q,k Q4_K + v Q6_K": synth.weight_nbytes(synth.Q4_K, 5120, 4096) + synth.weight_nbytes(synth.Q6_K, 1024, 4096),
                 "down Q4_K 4096x12288": synth.weight_nbytes(synth.Q4_K, 4096, 12288),
                 "down Q6_K 4096x12288": synth.weight_nbytes(synth.Q6_K, 4096, 12288),
                 "gate + up Q4_K 2 x 12288x4096": 2 * synth.weight_nbytes(synth.Q4_K, 12288, 4096)}
        for label, nbytes in sizes.items():
            span = (nbytes + 4095) // 4096 * 4096
            slots = total // span
            reps = 40
            for timed in (False, True):
                if timed:
                    capi.check(L.turq_profile_begin(ctx), ctx)
                for i in range(reps):
                    capi.check(L.turq_read_yardstick(ctx, ctypes.c_void_p(buf.value + (i % slots) * span), nbytes), ctx)
                if not timed:
                    capi.check(L.turq_sync(ctx), ctx)
            n, ms = ctypes.c_int64(), ctypes.c_double()
            capi.check(L.turq_profile_end(ctx, ctypes.byref(n), ctypes.byref(ms)), ctx)
            us = ms.value / max(1, n.value) * 1e3
            rows.append({"launch": label, "bytes": int(nbytes), "read_us": round(us, 2), "read_gbps": round(nbytes / us / 1e3, 1),
                         "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)})
    finally:
        if buf:
            L.turq_dev_free(ctx, buf)
        L.turq_ctx_destroy(ctx)
    return {"what": "a launch of the decode kernels' shape that only reads the same bytes (turq_read_yardstick), kernel time", "rows": rows}


def other_halves(base, b_mlp):
    """The rest of the headline metric, measured in the same process with the same method (value = whole step, frac = the
    matmul kernels alone against the peak of their bound), one entry per configuration of the metric: the MLP shapes at the
    other batch sizes and with bf16 activations (config 2) and as whole turq_mlp calls on prompt chunks, the prefill GEMM
    (config 4), the mixed Q4_K / Q6_K decoder layer at its batch sizes (config 3) and on prompt chunks, the Q6_K and Q5_K LM
    heads (config 5) and the small Q8_0 matrix that runs on the reference's CPU path today (config 1).  b_mlp: the headline's
    Bench, whose resident weights serve the legs on the same matrices."""
    steps, warmup = 20, 3
    out = {}
    out["q4k_mlp_f32"] = leg(b_mlp, [4, 16], "f32", "f32", steps, warmup)
    out["q4k_mlp_bf16"] = leg(b_mlp, [1, 4, 16], "bf16", "f32", steps, warmup)
    out["mlp_prefill"] = leg(b_mlp, [128, 512], "bf16", "bf16", 10, 2, mlp=True)
    plan = [
        ("q4k_prefill_up_8b", [("prefill", [512, 2048], "bf16", "bf16", steps, warmup)]),
        ("q4km_layer_8b", [("q4km_layer", [1, 8, 32], "f32", "f32", steps, warmup),
                           ("q4km_layer_bf16", [8, 32], "bf16", "f32", steps, warmup),
                           ("q4km_layer_prefill", [128, 512], "bf16", "bf16", 10, 2),
                           # the same layer with its norms and residual additions: the fused entry points against separate calls
                           ("q4km_layer_glue_fused", [1, 8], "f32", "f32", steps, warmup, "fused"),
                           ("q4km_layer_glue_separate", [1, 8], "f32", "f32", steps, warmup, "separate"),
                           ("q4km_layer_glue_fused_prefill", [128], "bf16", "bf16", 10, 2, "fused"),
                           ("q4km_layer_glue_separate_prefill", [128], "bf16", "bf16", 10, 2, "separate")]),
        ("lm_head_q6k_8b", [("lm_head_q6k", [1, 16, 128], "bf16", "f32", steps, warmup)]),
        ("lm_head_q5k_8b", [("lm_head_q5k", [1, 16, 128], "bf16", "f32", steps, warmup)]),
        ("q8_0_gate_0p6b", [("q8_0_gate", [1], "f32", "f32", steps, warmup)]),
    ]
    for workload, legs in plan:
        b = bench_for(base, workload)
        try:
            for key, ms, act, outdt, st, wu, *glue in legs:
                out[key] = leg(b, ms, act, outdt, st, wu, glue=glue[0] if glue else None)
        finally:
            b.close()
    for key in ("q4km_layer_glue_separate", "q4km_layer_glue_separate_prefill"):
        out[key]["note"] = "the two residual additions per layer are the engine's own launches in this form and are NOT made here; the fused form includes them"
    out["q8_0_gate"]["note"] = "3.3 MB of weights: the launch itself (about 4 us) bounds it, not the bytes"
    out["read_floor"] = read_floor()
    return out


if __name__ == "__main__":
    main()
