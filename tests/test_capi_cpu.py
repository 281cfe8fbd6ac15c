"""CPU-side checks of the C ABI: the library loads without a GPU, exports every symbol that
include/turq.h declares, and the parts that need no device (geometry, GGUF reader, error plumbing)
behave as the reference's interfaces do."""
import ctypes
import os
import re
import struct

import numpy as np
import pytest

from tur_amd import capi, synth
from tur_amd.gguf import write_gguf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "turq.h")).read()
    declared = set(re.findall(r"\b(turq_[a-z0-9_]+)\s*\(", header))
    L = capi.lib()
    missing = [s for s in sorted(declared) if not hasattr(L, s)]
    assert not missing, missing
    assert declared == set(capi.declared_symbols())      # the ctypes table binds exactly the header


def test_geometry_entry_points():
    L = capi.lib()
    assert L.turq_version().startswith(b"turq")
    assert [L.turq_block_bytes(d) for d in (Q8_0, Q4_K, Q5_K, Q6_K, 0, 1, 30, 99)] == [34, 144, 176, 210, 4, 2, 2, 0]
    assert L.turq_weight_nbytes(Q4_K, 12288, 4096) == 28_311_552
    assert L.turq_weight_nbytes(Q4_K, 4, 100) == 0                     # k not a multiple of 256
    assert L.turq_tiled_nbytes(Q4_K, 12288, 4096) == 28_311_552        # the tiled layout adds nothing here
    assert L.turq_tiled_nbytes(Q6_K, 17, 256) == 2 * 3360              # rows padded to 32


def test_context_errors_are_reported_not_raised():
    L = capi.lib()
    ctx = ctypes.c_void_p()
    assert L.turq_ctx_create(0, None) == capi.ERR_INVALID
    assert "null" in capi.last_error(None)
    assert L.turq_sync(None) == capi.ERR_INVALID
    if not os.path.exists("/dev/kfd"):
        rc = L.turq_ctx_create(0, ctypes.byref(ctx))
        assert rc != capi.OK and capi.last_error(None)                 # no GPU: a clear error, no crash, no CPU fallback
    assert L.turq_weight_release(None) == capi.OK
    assert L.turq_weight_retain(None) == capi.ERR_INVALID


@pytest.fixture()
def gguf_file(tmp_path):
    rng = np.random.default_rng(0)
    tensors = [
        ("blk.0.ffn_gate.weight", Q4_K, (48, 512), synth.random_weight(Q4_K, 48, 512, 1)),
        ("blk.0.attn_v.weight", Q6_K, (32, 256), synth.random_weight(Q6_K, 32, 256, 2)),
        ("blk.0.attn_q.weight", Q8_0, (16, 64), synth.random_weight(Q8_0, 16, 64, 3)),
        ("blk.0.attn_q.bias", 0, (16,), rng.standard_normal(16).astype("<f4").view(np.uint8)),
        ("output_norm.weight", 0, (512,), rng.standard_normal(512).astype("<f4").view(np.uint8)),
        ("token_embd.weight", Q5_K, (20, 256), synth.random_weight(Q5_K, 20, 256, 4)),
    ]
    meta = {"general.architecture": "qwen3", "qwen3.block_count": 1, "qwen3.rope.freq_base": 1000000.0,
            "tokenizer.ggml.tokens": ["a", "b", "c"], "general.file_type": 15}
    p = tmp_path / "tiny.gguf"
    write_gguf(str(p), tensors, meta)
    return str(p), tensors, meta


def test_gguf_reader(gguf_file):
    path, tensors, meta = gguf_file
    L = capi.lib()
    g = ctypes.c_void_p()
    capi.check(L.turq_gguf_open(path.encode(), ctypes.byref(g)))
    assert L.turq_gguf_tensor_count(g) == len(tensors)
    assert [L.turq_gguf_tensor_name(g, i).decode() for i in range(len(tensors))] == [t[0] for t in tensors]
    for name, dt, shape, raw in tensors:
        gdt, nd, nb, off = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t(), ctypes.c_uint64()
        dims = (ctypes.c_int64 * 4)()
        capi.check(L.turq_gguf_tensor_info(g, name.encode(), ctypes.byref(gdt), ctypes.byref(nd), dims, ctypes.byref(off), ctypes.byref(nb)))
        assert gdt.value == dt and tuple(dims[i] for i in range(nd.value)) == shape and nb.value == raw.size
        assert off.value % 32 == 0                                      # data section aligned to general.alignment
        buf = np.zeros(raw.size, np.uint8)
        capi.check(L.turq_gguf_read_tensor(g, name.encode(), capi.ptr(buf), buf.size))
        assert np.array_equal(buf, np.asarray(raw).view(np.uint8).reshape(-1))
    # metadata
    u, f = ctypes.c_uint64(), ctypes.c_double()
    capi.check(L.turq_gguf_meta_u64(g, b"qwen3.block_count", ctypes.byref(u)))
    assert u.value == 1
    capi.check(L.turq_gguf_meta_f64(g, b"qwen3.rope.freq_base", ctypes.byref(f)))
    assert f.value == 1000000.0
    s = ctypes.create_string_buffer(64)
    capi.check(L.turq_gguf_meta_str(g, b"general.architecture", s, 64))
    assert s.value == b"qwen3"
    capi.check(L.turq_gguf_meta_u64(g, b"tokenizer.ggml.tokens", ctypes.byref(u)))
    assert u.value == 3                                                 # arrays report their length
    assert L.turq_gguf_meta_u64(g, b"no.such.key", ctypes.byref(u)) == capi.ERR_NOT_FOUND
    assert L.turq_gguf_meta_u64(g, b"general.architecture", ctypes.byref(u)) == capi.ERR_DTYPE
    # lookups that miss
    assert L.turq_gguf_tensor_info(g, b"blk.9.nope", None, None, None, None, None) == capi.ERR_NOT_FOUND
    assert "cannot find tensor info" in L.turq_gguf_last_error(g).decode()
    small = np.zeros(8, np.uint8)
    assert L.turq_gguf_read_tensor(g, b"output_norm.weight", capi.ptr(small), small.size) == capi.ERR_SHAPE
    L.turq_gguf_close(g)


def test_gguf_reader_rejects_malformed_files(tmp_path):
    L = capi.lib()
    g = ctypes.c_void_p()
    assert L.turq_gguf_open(str(tmp_path / "missing.gguf").encode(), ctypes.byref(g)) == capi.ERR_IO
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"GGML" + b"\0" * 64)
    assert L.turq_gguf_open(str(bad).encode(), ctypes.byref(g)) == capi.ERR_IO and "magic" in capi.last_error(None)
    v9 = tmp_path / "v9.gguf"
    v9.write_bytes(struct.pack("<IIQQ", 0x46554747, 9, 0, 0))
    assert L.turq_gguf_open(str(v9).encode(), ctypes.byref(g)) == capi.ERR_IO and "version" in capi.last_error(None)
    trunc = tmp_path / "trunc.gguf"
    trunc.write_bytes(struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + struct.pack("<Q", 5) + b"ab")
    assert L.turq_gguf_open(str(trunc).encode(), ctypes.byref(g)) == capi.ERR_IO
    # innermost dimension not divisible by the block size
    ragged = tmp_path / "ragged.gguf"
    name = b"w"
    ragged.write_bytes(struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + struct.pack("<Q", 1) + name + struct.pack("<I", 2) +
                       struct.pack("<QQ", 100, 4) + struct.pack("<IQ", Q4_K, 0))
    assert L.turq_gguf_open(str(ragged).encode(), ctypes.byref(g)) == capi.ERR_IO and "block size" in capi.last_error(None)


def test_gguf_v2_and_alignment(tmp_path):
    # version 2 header (same field widths as v3) and a non-default general.alignment
    raw = synth.random_weight(Q8_0, 4, 32, 9)
    p = tmp_path / "al.gguf"
    write_gguf(str(p), [("a.weight", Q8_0, (4, 32), raw), ("b.weight", Q8_0, (4, 32), raw[::-1].copy())], {"k": 1}, alignment=64)
    data = bytearray(p.read_bytes())
    data[4:8] = struct.pack("<I", 2)
    p.write_bytes(bytes(data))
    L = capi.lib()
    g = ctypes.c_void_p()
    capi.check(L.turq_gguf_open(str(p).encode(), ctypes.byref(g)))
    off = ctypes.c_uint64()
    capi.check(L.turq_gguf_tensor_info(g, b"b.weight", None, None, None, ctypes.byref(off), None))
    assert off.value % 64 == 0
    buf = np.zeros(raw.size, np.uint8)
    capi.check(L.turq_gguf_read_tensor(g, b"b.weight", capi.ptr(buf), buf.size))
    assert np.array_equal(buf, raw[::-1])
    L.turq_gguf_close(g)


# ---- a GGUF file assembled by hand from the published layout (not by tur_amd.gguf), and hostile variants of it ----
def _gguf_v3_bytes(tensor_offset_1=None, dup=False, str_len=None, arr_len=None):
    import struct

    def s(b):
        return struct.pack("<Q", len(b)) + b

    q8 = bytes(range(34)) * 2                       # one row of two Q8_0 blocks: [1, 64]
    f32 = struct.pack("<6f", 1.0, 2.0, 3.0, 4.0, 5.0, 6.0)      # [2, 3] row-major
    head = b"GGUF" + struct.pack("<I", 3) + struct.pack("<QQ", 2, 3)
    # metadata: one string, one u32, one array of three i32
    head += s(b"general.architecture") + struct.pack("<I", 8) + (struct.pack("<Q", str_len) + b"qwen3" if str_len is not None else s(b"qwen3"))
    head += s(b"qwen3.block_count") + struct.pack("<II", 4, 36)
    head += s(b"some.list") + struct.pack("<IIQ", 9, 5, 3 if arr_len is None else arr_len) + struct.pack("<3i", 7, 8, 9)
    # tensor infos: name, n_dims, dims innermost first, ggml dtype, offset into the data section
    head += s(b"blk.0.w") + struct.pack("<I", 2) + struct.pack("<QQ", 64, 1) + struct.pack("<IQ", 8, 0)
    second = b"blk.0.w" if dup else b"norm.weight"
    head += s(second) + struct.pack("<I", 2) + struct.pack("<QQ", 3, 2) + struct.pack("<IQ", 0, 96 if tensor_offset_1 is None else tensor_offset_1)
    pad = (-len(head)) % 32
    data = q8 + b"\0" * (96 - len(q8)) + f32          # second tensor at the next multiple of 32 after 68 bytes
    return head + b"\0" * pad + data, len(head) + pad, q8, f32


def test_gguf_reader_on_a_hand_assembled_file(tmp_path):
    L = capi.lib()
    blob, data_off, q8, f32 = _gguf_v3_bytes()
    p = tmp_path / "hand.gguf"
    p.write_bytes(blob)
    g = ctypes.c_void_p()
    assert L.turq_gguf_open(str(p).encode(), ctypes.byref(g)) == capi.OK, capi.last_error()
    assert L.turq_gguf_tensor_count(g) == 2
    assert [L.turq_gguf_tensor_name(g, i) for i in range(2)] == [b"blk.0.w", b"norm.weight"]
    dt, nd, off, nb = ctypes.c_int(), ctypes.c_int(), ctypes.c_uint64(), ctypes.c_size_t()
    dims = (ctypes.c_int64 * 4)()
    assert L.turq_gguf_tensor_info(g, b"blk.0.w", ctypes.byref(dt), ctypes.byref(nd), dims, ctypes.byref(off), ctypes.byref(nb)) == capi.OK
    assert (dt.value, nd.value, dims[0], dims[1], off.value, nb.value) == (capi.Q8_0, 2, 1, 64, data_off, 68)      # (n, k): GGUF order reversed
    assert L.turq_gguf_tensor_info(g, b"norm.weight", ctypes.byref(dt), ctypes.byref(nd), dims, ctypes.byref(off), ctypes.byref(nb)) == capi.OK
    assert (dt.value, nd.value, dims[0], dims[1], off.value, nb.value) == (capi.F32, 2, 2, 3, data_off + 96, 24)
    buf = ctypes.create_string_buffer(68)
    assert L.turq_gguf_read_tensor(g, b"blk.0.w", buf, 68) == capi.OK and buf.raw == q8
    buf = ctypes.create_string_buffer(24)
    assert L.turq_gguf_read_tensor(g, b"norm.weight", buf, 24) == capi.OK and buf.raw == f32
    v = ctypes.c_uint64()
    assert L.turq_gguf_meta_u64(g, b"qwen3.block_count", ctypes.byref(v)) == capi.OK and v.value == 36
    assert L.turq_gguf_meta_u64(g, b"some.list", ctypes.byref(v)) == capi.OK and v.value == 3      # arrays report their length
    name = ctypes.create_string_buffer(32)
    assert L.turq_gguf_meta_str(g, b"general.architecture", name, 32) == capi.OK and name.value == b"qwen3"
    L.turq_gguf_close(g)


@pytest.mark.parametrize("kwargs,what", [
    (dict(tensor_offset_1=2**64 - 8), "runs past the end"),        # offset + size wraps around 2^64
    (dict(tensor_offset_1=10**6), "runs past the end"),
    (dict(dup=True), "listed twice"),
    (dict(str_len=2**40), "runs past the end"),                    # a string longer than the file
    (dict(arr_len=2**62), "runs past the end"),                    # array length * element size wraps
], ids=["offset-wraps", "offset-beyond", "duplicate-name", "string-length", "array-length"])
def test_gguf_reader_refuses_hostile_files(tmp_path, kwargs, what):
    L = capi.lib()
    blob = _gguf_v3_bytes(**kwargs)[0]
    p = tmp_path / "bad.gguf"
    p.write_bytes(blob)
    g = ctypes.c_void_p()
    rc = L.turq_gguf_open(str(p).encode(), ctypes.byref(g))
    if rc == capi.OK:          # the header parses; the tensor whose bytes are not there must be refused on read
        buf = ctypes.create_string_buffer(24)
        assert L.turq_gguf_read_tensor(g, b"norm.weight", buf, 24) == capi.ERR_IO
        assert what in L.turq_gguf_last_error(g).decode()
        L.turq_gguf_close(g)
    else:
        assert rc == capi.ERR_IO and what in capi.last_error()


def test_prefill_launch_rules_on_a_256_cu_device():
    # the launches the rules make for the matrices of a Qwen3-8B Q4_K_M layer on prompt chunks, as measured and documented:
    # (tile, workgroups per tile, wave groups); tiles: 1 = 128 x 128, 2 = 128 x 192, 3 = 128 x 256, 4 = 64 x 128
    L = capi.lib()
    Q4_K, Q6_K = capi.Q4_K, capi.Q6_K

    def plan(dt, n, k, m):
        t, s, g = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        capi.check(L.turq_prefill_plan(dt, n, k, m, 256, ctypes.byref(t), ctypes.byref(s), ctypes.byref(g)))
        return t.value, s.value, g.value

    # down_proj 4096 x 12288: low tile in 6 / 3 parts up to 128 rows, wide tile in 6 parts at 256, unsplit from 512 on
    assert plan(Q6_K, 4096, 12288, 64) == (4, 6, 2)
    assert plan(Q6_K, 4096, 12288, 128) == (4, 3, 2)
    assert plan(Q6_K, 4096, 12288, 256) == (3, 6, 1)
    assert plan(Q6_K, 4096, 12288, 512) == (4, 1, 2)
    assert plan(Q6_K, 4096, 12288, 1024) == (1, 1, 1)
    # o_proj / q_proj 4096 x 4096 and k_proj 1024 x 4096: parts only while they take at most a quarter of the CUs; eight waves
    # while there is at most one workgroup per CU
    assert plan(Q4_K, 4096, 4096, 64) == (4, 2, 2)
    assert plan(Q4_K, 4096, 4096, 128) == (4, 1, 2)
    assert plan(Q4_K, 1024, 4096, 128) == (4, 4, 2)
    assert plan(Q4_K, 4096, 4096, 256) == (4, 1, 2)
    assert plan(Q4_K, 4096, 4096, 512) == (4, 1, 2)
    # up_proj 12288 x 4096 alone, and gate + up as one launch (24576 rows)
    assert plan(Q4_K, 12288, 4096, 128) == (4, 1, 2)
    assert plan(Q4_K, 12288, 4096, 256) == (1, 1, 1)
    assert plan(Q4_K, 12288, 4096, 512) == (2, 1, 1)
    assert plan(Q4_K, 12288, 4096, 2048) == (3, 1, 1)
    assert plan(Q4_K, 24576, 4096, 128) == (1, 1, 1)
    assert plan(Q4_K, 24576, 4096, 256) == (2, 1, 1)
    assert plan(Q4_K, 24576, 4096, 1024) == (3, 1, 1)
    # the LM head: more workgroups than CUs, four waves
    assert plan(Q6_K, 151936, 4096, 64) == (4, 1, 1)
    # gate_proj and up_proj (2 x 12288 x 4096) through turq_qmatmul_multi: one launch where that fills the rounds better, which the
    # timings behind the rule show at 128, 256 and 1024 rows and not at 384 and 512; k_proj and v_proj are too small to merge
    def merged(n, m, cus, count=2):
        g = ctypes.c_int(-1)
        capi.check(L.turq_prefill_plan_multi(Q4_K, n, 4096, m, count, cus, ctypes.byref(g)))
        return g.value

    assert [merged(12288, m, 256) for m in (64, 128, 256, 384, 512, 1024, 2048)] == [0, 1, 1, 0, 0, 1, 0]
    assert [merged(1024, m, 256) for m in (64, 256, 2048)] == [0, 0, 0]
    assert merged(12288, 256, 256, count=1) == 0
    # the rule counts rounds over the CUs, so a device of half the size decides differently at the same shapes
    assert [merged(12288, m, 128) for m in (64, 128, 256, 384, 512, 1024, 2048)] == [0, 1, 0, 1, 1, 0, 0]
    assert merged(1024, 2048, 128) == 1
    # arguments
    t = ctypes.c_int()
    assert L.turq_prefill_plan_multi(Q4_K, 12288, 4096, 8, 2, 256, ctypes.byref(t)) == capi.ERR_SHAPE
    assert L.turq_prefill_plan_multi(Q4_K, 12288, 4096, 64, 5, 256, ctypes.byref(t)) == capi.ERR_SHAPE
    assert L.turq_prefill_plan_multi(capi.F32, 12288, 4096, 64, 2, 256, ctypes.byref(t)) == capi.ERR_DTYPE
    assert L.turq_prefill_plan(Q4_K, 4096, 4096, 8, 256, ctypes.byref(t), None, None) == capi.ERR_SHAPE
    assert L.turq_prefill_plan(capi.F32, 4096, 4096, 64, 256, ctypes.byref(t), None, None) == capi.ERR_DTYPE



def test_tuning_switches_are_listed_and_overrides_are_announced():
    # every environment switch of the kernel-selection rules lives in one table (tur_amd/csrc/tuning.h); a process lists what it
    # runs with, and says on stderr when any of them is set
    import os
    import re
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    names = re.findall(r'X\(\w+, "(TURQ_\w+)"', open(os.path.join(root, "tur_amd", "csrc", "tuning.h")).read())
    assert len(names) >= 25 and len(set(names)) == len(names)
    # no other source file of the library reads the environment for a TURQ_ variable
    for dirpath, _, files in os.walk(os.path.join(root, "tur_amd", "csrc")):
        for f in files:
            if f.endswith((".cpp", ".hip", ".h", ".hpp")) and f not in ("tuning.cpp", "tuning.h"):
                assert not re.search(r'getenv\("TURQ_', open(os.path.join(dirpath, f)).read()), f
    code = ("import ctypes\nfrom tur_amd import capi\nL = capi.lib()\nn = ctypes.c_size_t()\n"
            "capi.check(L.turq_tuning_describe(None, 0, ctypes.byref(n)))\nb = ctypes.create_string_buffer(n.value)\n"
            "capi.check(L.turq_tuning_describe(b, n.value, None))\nprint(b.value.decode())\n")
    env = {k: v for k, v in os.environ.items() if not k.startswith("TURQ_")}
    plain = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, check=True)
    lines = plain.stdout.strip().splitlines()
    assert [ln.split("=")[0] for ln in lines] == names
    assert all("(default)" in ln for ln in lines) and "libturq" not in plain.stderr
    env.update(TURQ_GEMM_WIDE="0", TURQ_GEMV_NO_ROW1="1")
    forced = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, check=True)
    assert "2 kernel-selection override(s) from the environment: TURQ_GEMV_NO_ROW1=1 TURQ_GEMM_WIDE=0" in forced.stderr
    by = {ln.split("=")[0]: ln for ln in forced.stdout.strip().splitlines()}
    assert by["TURQ_GEMM_WIDE"].startswith("TURQ_GEMM_WIDE=0  (set)") and by["TURQ_GEMV_NO_ROW1"].startswith("TURQ_GEMV_NO_ROW1=1  (set)")
    assert by["TURQ_GEMM_LOW"].startswith("TURQ_GEMM_LOW=-1  (default)")
