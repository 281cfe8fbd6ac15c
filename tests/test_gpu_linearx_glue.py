"""The host mirrors of the decoder layer's glue: LinearX.forward_add, NormX.forward_then, NormX.forward_mlp_residual and
Device.nonfinite_count of tur_amd.qlinear (host arrays through the C ABI, the way the reference's layers see tensors:
src/models/qwen3.rs:633-640), against the f64 formulas on the oracle's dequantized weights."""
import numpy as np
import pytest

from oracle import capi as orc
from oracle import oracle_np as onp
from tests.helpers import rel_l2
from tur_amd import capi, qlinear, synth

pytestmark = pytest.mark.gpu
Q4_K, Q6_K = capi.Q4_K, capi.Q6_K


def want_norm(x, w, eps):
    x64 = np.asarray(x, np.float64)
    return (x64 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + eps) * np.asarray(w, np.float64)).astype(np.float32)


def test_a_decoder_layer_without_attention():
    dev = qlinear.Device(0)
    hid, kv, ff, eps = 1024, 256, 2048, 1e-6
    rng = np.random.default_rng(3)
    shapes = {"q": (Q4_K, hid, hid), "k": (Q4_K, kv, hid), "v": (Q6_K, kv, hid), "o": (Q4_K, hid, hid), "gate": (Q4_K, ff, hid),
              "up": (Q4_K, ff, hid), "down": (Q6_K, hid, ff)}
    raws = {nm: synth.random_weight(dt, n, k, seed=i) for i, (nm, (dt, n, k)) in enumerate(shapes.items())}
    lin = {nm: qlinear.LinearX(qlinear.QMatMul.from_arc(qlinear.QTensor.new(dev, dt, (n, k), raws[nm]))) for nm, (dt, n, k) in shapes.items()}
    ln1 = qlinear.NormX(dev, 1.0 + 0.1 * rng.standard_normal(hid).astype(np.float32), eps)
    ln2 = qlinear.NormX(dev, 0.02 * (1.0 + 0.1 * rng.standard_normal(hid)).astype(np.float32), eps)
    for m in (1, 5, 40):
        x = (rng.standard_normal((m, hid)) * 3).astype(np.float32)
        attn = rng.standard_normal((m, hid)).astype(np.float32)            # stands for the attention block's output
        dev.nonfinite_count()
        q, k, v = ln1.forward_then([lin[nm].qmatmul for nm in ("q", "k", "v")], x)
        xn = want_norm(x, ln1.weight, eps)
        for nm, y in (("q", q), ("k", k), ("v", v)):
            dt, n, kk = shapes[nm]
            assert rel_l2(y, orc.matmul_dequant(dt, xn, raws[nm], n, kk)) <= 1e-3, (nm, m)
        x1 = lin["o"].forward_add(attn, x)                                  # x + o_proj(attn)
        want1 = x + orc.matmul_dequant(Q4_K, attn, raws["o"], hid, hid)
        assert rel_l2(x1 - x, want1 - x) <= 1e-3
        x2 = ln2.forward_mlp_residual(lin["gate"].qmatmul, lin["up"].qmatmul, lin["down"].qmatmul, x1)
        xn2 = want_norm(x1, ln2.weight, eps)
        h = onp.silu_mul(orc.matmul_dequant(Q4_K, xn2, raws["gate"], ff, hid), orc.matmul_dequant(Q4_K, xn2, raws["up"], ff, hid))
        want2 = x1 + orc.matmul_dequant(Q6_K, h, raws["down"], hid, ff)
        assert rel_l2(x2 - x1, want2 - x1) <= 2e-3, (m, rel_l2(x2 - x1, want2 - x1))
        assert dev.nonfinite_count() == 0
    with pytest.raises(qlinear.TurqError):
        lin["o"].forward_add(attn, np.zeros((3, 7), np.float32))
    with pytest.raises(qlinear.TurqError):
        ln1.forward_then([lin["down"].qmatmul], x)
    dev.close()
