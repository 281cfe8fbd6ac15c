"""GPU tests of the host-side mirror (QVarBuilder / QMatMul / LinearX), written the way the reference
tests its own layer (src/models/layers/linear.rs:117-316: shapes, batch shapes, bias, clone) and its
integration tests check the quantized path (tests/qwen3_integration.rs: shape, finiteness,
single-vs-batched consistency), with the numeric parity the reference's tests lack."""
import numpy as np
import pytest

from oracle import capi as orc
from tests.helpers import rel_l2
from tur_amd import capi, qlinear, synth
from tur_amd.gguf import write_gguf

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
HID, FFN, KV = 512, 1536, 256


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    """one synthetic decoder layer in the Q4_K_M mix + a biased projection + an F32 norm"""
    rng = np.random.default_rng(5)
    spec = [("blk.0.attn_q.weight", Q4_K, (HID, HID)), ("blk.0.attn_k.weight", Q4_K, (KV, HID)),
            ("blk.0.attn_v.weight", Q6_K, (KV, HID)), ("blk.0.attn_output.weight", Q4_K, (HID, HID)),
            ("blk.0.ffn_gate.weight", Q4_K, (FFN, HID)), ("blk.0.ffn_up.weight", Q4_K, (FFN, HID)),
            ("blk.0.ffn_down.weight", Q6_K, (HID, FFN)), ("output.weight", Q8_0, (1000, HID)),
            ("blk.0.biased.weight", Q5_K, (96, HID))]
    tensors = [(name, dt, shape, synth.random_weight(dt, shape[0], shape[1], seed=i)) for i, (name, dt, shape) in enumerate(spec)]
    bias = rng.standard_normal(96).astype("<f4")
    norm = rng.standard_normal(HID).astype("<f4")
    tensors += [("blk.0.biased.bias", 0, (96,), bias.view(np.uint8)), ("blk.0.attn_norm.weight", 0, (HID,), norm.view(np.uint8))]
    path = tmp_path_factory.mktemp("gguf") / "layer.gguf"
    write_gguf(str(path), tensors, {"general.architecture": "qwen3"})
    dev = qlinear.Device.new_hip(0)
    vb = qlinear.QVarBuilder.from_gguf(str(path), dev)
    yield dev, vb, {t[0]: t for t in tensors}, bias, norm
    dev.close()


def test_varbuilder_lookups(model):
    dev, vb, tensors, _, _ = model
    assert sorted(vb.all_keys()) == sorted(tensors)
    b0 = vb.pp("blk").pp(0)
    assert b0.path("attn_q.weight") == "blk.0.attn_q.weight"
    assert b0.contains_key("attn_q.weight") and not b0.contains_key("attn_q.bias")
    assert b0.tensor_shape("ffn_down.weight") == [HID, FFN] and b0.tensor_shape("nope") is None
    t = b0.pp("attn_k").get((KV, HID), "weight")
    assert t.shape() == (KV, HID) and t.dtype() == Q4_K
    with pytest.raises(capi.TurqError, match="shape mismatch for weight"):
        b0.pp("attn_k").get((HID, HID), "weight")          # cached tensor, wrong shape
    with pytest.raises(capi.TurqError, match="shape mismatch for weight"):
        b0.pp("attn_v").get((HID, HID), "weight")          # fresh tensor, wrong shape
    with pytest.raises(capi.TurqError, match="cannot find tensor info"):
        b0.pp("attn_x").get((HID, HID), "weight")
    assert b0.get_no_shape("attn_norm.weight").shape() == (HID,)


def test_norm_weight_dequantizes_like_the_reference(model):
    dev, vb, _, _, norm = model
    got = vb.pp("blk").pp(0).pp("attn_norm").get(HID, "weight").dequantize(dev)
    assert got.shape == (HID,) and np.array_equal(got, norm)


@pytest.mark.parametrize("name,out_dim,in_dim", [("attn_q", HID, HID), ("attn_k", KV, HID), ("attn_v", KV, HID),
                                                 ("attn_output", HID, HID), ("ffn_gate", FFN, HID), ("ffn_up", FFN, HID),
                                                 ("ffn_down", HID, FFN)])
def test_decoder_layer_linears(model, name, out_dim, in_dim):
    dev, vb, tensors, _, _ = model
    layer = qlinear.linear(in_dim, out_dim, vb.pp("blk").pp(0).pp(name))
    assert repr(layer) == "LinearX::Quantized" and layer.bias is None
    _, dt, _, raw = tensors[f"blk.0.{name}.weight"]
    rng = np.random.default_rng(0)
    for shape in ((1, 1, in_dim), (2, 5, in_dim), (1, 40, in_dim)):      # [batch, seq, hidden] as the models call it
        x = rng.standard_normal(shape).astype(np.float32)
        y = layer.forward(x)
        assert y.shape == shape[:-1] + (out_dim,) and np.all(np.isfinite(y))
        want = orc.matmul_dequant(dt, x.reshape(-1, in_dim), raw, out_dim, in_dim).reshape(y.shape)
        assert rel_l2(y, want) <= 1e-3
    # single vs batched: row 0 of a batch equals the same row alone (the reference allows 1e-2 here)
    xb = rng.standard_normal((3, 1, in_dim)).astype(np.float32)
    yb = layer.forward(xb)
    y0 = layer.forward(xb[0:1])
    assert np.max(np.abs(yb[0] - y0[0])) <= 1e-3 * np.max(np.abs(y0))


def test_qkv_projections_in_one_call(model):
    # the reference applies q_proj, k_proj and v_proj to the same hidden state back to back (qwen3.rs:272-274)
    dev, vb, tensors, _, _ = model
    names = [("attn_q", HID), ("attn_k", KV), ("attn_v", KV)]
    layers = [qlinear.linear(HID, out, vb.pp("blk").pp(0).pp(nm)) for nm, out in names]
    x = np.random.default_rng(5).standard_normal((1, 2, HID)).astype(np.float32)
    ys = qlinear.QMatMul.forward_multi([l.qmatmul for l in layers], x)
    for (nm, out), layer, y in zip(names, layers, ys):
        assert y.shape == (1, 2, out)
        assert np.array_equal(y, layer.forward(x))          # host tensors: literally the single calls
    with pytest.raises(capi.TurqError):
        qlinear.QMatMul.forward_multi([l.qmatmul for l in layers], x[..., :-1].copy())


def test_mlp_gate_up_in_one_call(model):
    # Qwen3MLP::forward, first half (qwen3.rs:161-167): silu(gate_proj(x)) * up_proj(x)
    dev, vb, tensors, _, _ = model
    gate = qlinear.linear(HID, FFN, vb.pp("blk").pp(0).pp("ffn_gate"))
    up = qlinear.linear(HID, FFN, vb.pp("blk").pp(0).pp("ffn_up"))
    x = (np.random.default_rng(6).standard_normal((2, 3, HID)) / 64).astype(np.float32)
    y = qlinear.QMatMul.forward_gate_up(gate.qmatmul, up.qmatmul, x)
    assert y.shape == (2, 3, FFN)
    g, u = gate.forward(x).astype(np.float64), up.forward(x).astype(np.float64)
    assert rel_l2(y, (g / (1 + np.exp(-g)) * u).astype(np.float32)) <= 1e-6
    with pytest.raises(capi.TurqError):
        qlinear.QMatMul.forward_gate_up(gate.qmatmul, up.qmatmul, x[..., :-1].copy())
    down = qlinear.linear(FFN, HID, vb.pp("blk").pp(0).pp("ffn_down"))
    with pytest.raises(capi.TurqError):       # gate and up of different shapes
        qlinear.QMatMul.forward_gate_up(gate.qmatmul, down.qmatmul, x)
    # the whole of Qwen3MLP::forward through one call: down_proj of that product
    z = qlinear.QMatMul.forward_mlp(gate.qmatmul, up.qmatmul, down.qmatmul, x)
    assert z.shape == (2, 3, HID)
    assert rel_l2(z, down.forward(y)) <= 1e-6
    with pytest.raises(capi.TurqError):       # down_proj must take what gate / up give
        qlinear.QMatMul.forward_mlp(gate.qmatmul, up.qmatmul, gate.qmatmul, x)


def test_embedding_over_the_quantized_table(model):
    # layers::embedding (layers/mod.rs:11-50): table [vocab, hidden], forward(ids) -> ids.shape + [hidden]
    dev, vb, tensors, _, _ = model
    emb, vocab = qlinear.embedding(None, HID, vb.pp("output"))          # the 1000 x 512 Q8_0 tensor of the fixture
    assert vocab == 1000
    emb2, vocab2 = qlinear.embedding(1000, HID, vb.pp("output"))
    assert vocab2 == 1000
    with pytest.raises(capi.TurqError):
        qlinear.embedding(999, HID, vb.pp("output"))                    # shape mismatch as in gguf_varbuilder.rs:62-66
    ids = np.array([[0, 999, 7], [7, 7, 3]])
    y = emb.forward(ids)
    assert y.shape == (2, 3, HID)
    raw = tensors["output.weight"][3]
    table = orc.dequantize(Q8_0, raw).reshape(1000, HID)
    assert np.array_equal(y, table[ids])
    assert np.array_equal(emb2.forward(ids), y)
    with pytest.raises(capi.TurqError):
        emb.forward(np.array([1000]))


def test_bias_is_dequantized_at_load_and_added(model):
    dev, vb, tensors, bias, _ = model
    layer = qlinear.linear(HID, 96, vb.pp("blk").pp(0).pp("biased"))
    assert layer.bias is not None and np.array_equal(layer.bias, bias)
    x = np.zeros((1, 2, HID), np.float32)
    assert np.array_equal(layer.forward(x), np.broadcast_to(bias, (1, 2, 96)))      # zero input -> bias
    x = np.random.default_rng(1).standard_normal((1, 3, HID)).astype(np.float32)
    _, dt, _, raw = tensors["blk.0.biased.weight"]
    want = orc.matmul_dequant(dt, x.reshape(-1, HID), raw, 96, HID).reshape(1, 3, 96) + bias
    assert rel_l2(layer.forward(x), want) <= 1e-3


def test_lm_head_and_clone(model):
    dev, vb, tensors, _, _ = model
    head = qlinear.linear(HID, 1000, vb.pp("output"))
    clone = qlinear.LinearX(qlinear.QMatMul.from_arc(head.qmatmul.qtensor.clone()), None)
    head.qmatmul.qtensor.release()                                     # the clone keeps the device copy alive
    x = np.random.default_rng(2).standard_normal((1, 1, HID)).astype(np.float32)
    y = clone.forward(x)
    _, dt, _, raw = tensors["output.weight"]
    assert y.shape == (1, 1, 1000)
    assert rel_l2(y, orc.matmul_dequant(dt, x.reshape(1, HID), raw, 1000, HID).reshape(1, 1, 1000)) <= 1e-3


def test_forward_argument_errors(model):
    dev, vb, _, _, _ = model
    layer = qlinear.linear(HID, KV, vb.pp("blk").pp(0).pp("attn_k"))
    with pytest.raises(capi.TurqError):
        layer.forward(np.zeros(HID, np.float32))                        # rank < 2
    with pytest.raises(capi.TurqError):
        layer.forward(np.zeros((1, HID + 1), np.float32))               # last dim != k
    with pytest.raises(capi.TurqError):
        layer.forward(np.zeros((2, 4, HID), np.float32)[:, ::2, :])     # not contiguous
    with pytest.raises(capi.TurqError):
        layer.forward(np.zeros((1, HID), np.float64))                   # unsupported dtype
    assert qlinear.QMatMul.from_arc(vb.pp("blk").pp(0).pp("attn_norm").get(HID, "weight")).dense   # a dense tensor: the dense arm
    assert layer.forward(np.zeros((0, HID), np.float32)).shape == (0, KV)   # empty batch


def test_cpp_host_mirror(model, tmp_path):
    """the C++ header mirror (tur_amd/csrc/host/turq.hpp) run as a program against the same kind of file"""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "test_host")
    if not os.path.exists(exe):
        pytest.fail("tests/cpp/test_host is not built (run __graft_entry__.build())")
    rng = np.random.default_rng(11)
    n, k = 160, 512
    gate = synth.random_weight(Q4_K, n, k, seed=1)
    biased = synth.random_weight(Q6_K, 96, k, seed=2)
    bias = rng.standard_normal(96).astype("<f4")
    norm = rng.standard_normal(k).astype("<f4")
    down = synth.random_weight(Q8_0, 64, n, seed=3)
    path = tmp_path / "cpp.gguf"
    write_gguf(str(path), [("blk.0.ffn_gate.weight", Q4_K, (n, k), gate), ("blk.0.biased.weight", Q6_K, (96, k), biased),
                           ("blk.0.ffn_down.weight", Q8_0, (64, n), down),
                           ("blk.0.biased.bias", 0, (96,), bias.view(np.uint8)), ("blk.0.attn_norm.weight", 0, (k,), norm.view(np.uint8))])
    res = subprocess.run([exe, str(path)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    lines = res.stdout.split("\n")
    assert lines[-2] == "OK"
    m = 3
    x = (np.sin(np.float32(0.37) * np.arange(m * k, dtype=np.float32)) * np.float32(2.0)).astype(np.float32).reshape(m, k)
    i = lines.index(f"gate {n} {k}")
    y = np.array([float(v) for v in lines[i + 1:i + 1 + m * n]], np.float32).reshape(m, n)
    j = lines.index(f"biased 96 {k}")
    yb = np.array([float(v) for v in lines[j + 1:j + 1 + m * 96]], np.float32).reshape(m, 96)
    assert rel_l2(y, orc.matmul_dequant(Q4_K, x, gate, n, k)) <= 1e-3
    assert rel_l2(yb, orc.matmul_dequant(Q6_K, x, biased, 96, k) + bias) <= 1e-3
    assert lines[-3].startswith(f"norm {k} ")


# ---- the dense arm of QMatMul::from_arc (src/models/layers/linear.rs:69 -> candle: F32 / F16 / BF16 tensors, and every
# tensor under CANDLE_DEQUANTIZE_ALL, become a dense f32 matmul on the dequantized weights) ----
def _dense_raw(dt, n, k, seed):
    w = np.random.default_rng(seed).standard_normal((n, k)).astype(np.float32) * 0.05
    if dt == capi.F32:
        return w.view(np.uint8).reshape(-1)
    if dt == capi.F16:
        return w.astype(np.float16).view(np.uint8).reshape(-1)
    return synth.to_bf16_bits(w).view(np.uint8).reshape(-1)


@pytest.mark.parametrize("dt", [capi.F32, capi.F16, capi.BF16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("n,k", [(96, 512), (33, 100), (7, 4099), (1, 5)])
def test_dense_weights_take_the_dense_matmul(model, dt, n, k):
    dev = model[0]
    raw = _dense_raw(dt, n, k, seed=n + k)
    layer = qlinear.LinearX(qlinear.QMatMul.from_arc(qlinear.QTensor.new(dev, dt, (n, k), raw)))
    assert layer.qmatmul.dense
    rng = np.random.default_rng(1)
    for shape in ((1, 1, k), (2, 5, k), (1, 40, k)):
        x = (rng.standard_normal(shape) * 3).astype(np.float32)
        y = layer.forward(x)
        want = orc.matmul_dequant(dt, x.reshape(-1, k), raw, n, k).reshape(y.shape)
        assert y.shape == shape[:-1] + (n,)
        assert rel_l2(y, want) <= 2e-6        # f32 products and sums against the f64 sum: no activation rounding


def test_dense_weight_from_a_gguf_file_and_activation_range(model, tmp_path):
    dev = model[0]
    n, k = 48, 256
    raw16 = _dense_raw(capi.F16, n, k, seed=3)
    bias = np.random.default_rng(4).standard_normal(n).astype("<f4")
    path = tmp_path / "dense.gguf"
    write_gguf(str(path), [("output.weight", capi.F16, (n, k), raw16), ("output.bias", 0, (n,), bias.view(np.uint8))])
    vb = qlinear.QVarBuilder.from_gguf(str(path), dev)
    layer = qlinear.linear(k, n, vb.pp("output"))
    assert layer.qmatmul.dense and np.array_equal(layer.bias, bias)
    # the dense arm computes in f32: activations far outside the f16 range are fine
    x = (np.random.default_rng(5).standard_normal((3, k)) * 1e6).astype(np.float32)
    want = orc.matmul_dequant(capi.F16, x, raw16, n, k) + bias
    assert rel_l2(layer.forward(x), want) <= 2e-6


@pytest.mark.parametrize("dt", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_dequantize_all_switch(model, dt, monkeypatch):
    # CANDLE_DEQUANTIZE_ALL: the quantized tensor becomes a dense f32 matmul on its dequantized values
    dev = model[0]
    n, k = 80, 1024
    raw = synth.random_weight(dt, n, k, seed=dt)
    qt = qlinear.QTensor.new(dev, dt, (n, k), raw)              # tiled, as the loader uploads matmul weights
    x = np.random.default_rng(6).standard_normal((5, k)).astype(np.float32)
    want = orc.matmul_dequant(dt, x, raw, n, k)
    quantized = qlinear.QMatMul.from_arc(qt)
    assert not quantized.dense
    monkeypatch.setenv("CANDLE_DEQUANTIZE_ALL", "1")
    dense = qlinear.QMatMul.from_arc(qt)
    assert dense.dense
    err_dense, err_quant = rel_l2(dense.forward(x), want), rel_l2(quantized.forward(x), want)
    assert err_dense <= 2e-6 and err_quant <= 1e-3 and err_dense < err_quant
