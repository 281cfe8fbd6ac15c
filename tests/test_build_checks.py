"""The build-time checker of the prefill GEMM's hand-placed LDS waits (tur_amd/csrc/check_lds_waits.py), on small
hand-written assembly snippets: a use before the covering wait is reported, the same use after it is not."""
import importlib.util
import os

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("check_lds_waits", os.path.join(HERE, "..", "tur_amd", "csrc", "check_lds_waits.py"))
chk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(chk)


def run(body):
    text = ["_Z4kernv:"] + ["\t" + ln for ln in body] + ["\ts_endpgm"]
    errs = []
    for name, ins in chk.kernel_bodies(text, "kern"):
        errs += chk.check_body(name, ins)
    return errs


def test_use_after_wait_is_clean():
    assert run(["ds_read_b128 v[4:7], v1 offset:16", "s_waitcnt lgkmcnt(0)", "v_mov_b32_e32 v9, v5"]) == []


def test_use_before_wait_is_reported():
    errs = run(["ds_read_b128 v[4:7], v1 offset:16", "v_mov_b32_e32 v9, v5", "s_waitcnt lgkmcnt(0)"])
    assert len(errs) >= 1 and "v_mov_b32_e32 v9, v5" in errs[0]


def test_overwrite_before_wait_is_reported():
    assert run(["ds_read_b128 v[4:7], v1", "v_mov_b32_e32 v6, 0", "s_waitcnt lgkmcnt(0)"])


def test_partial_wait_completes_the_oldest_reads_only():
    body = ["ds_read_b128 v[4:7], v1", "ds_read_b128 v[8:11], v1 offset:1024", "s_waitcnt lgkmcnt(1)"]
    assert run(body + ["v_add_u32_e32 v20, v4, v5"]) == []
    assert run(body + ["v_add_u32_e32 v20, v8, v5"])


def test_wait_without_the_lds_counter_completes_nothing():
    assert run(["ds_read_b32 v4, v1", "s_waitcnt vmcnt(0)", "v_mov_b32_e32 v9, v4"])


def test_scalar_load_outstanding_needs_a_full_wait():
    body = ["ds_read_b32 v4, v1", "s_load_dword s4, s[0:1], 0x0", "s_waitcnt lgkmcnt(1)", "v_mov_b32_e32 v9, v4"]
    assert run(body)


def test_loop_back_edge_is_walked():
    # the read at the bottom of the loop is used at its top on the next trip, without a wait in between
    body = [".LBB0_1:", "v_mov_b32_e32 v9, v4", "s_waitcnt lgkmcnt(0)", "ds_read_b32 v4, v1", "s_cbranch_scc1 .LBB0_1", "s_waitcnt lgkmcnt(0)"]
    assert run(body)


def test_resource_remarks(tmp_path):
    p = tmp_path / "r.txt"
    p.write_text("x.hip:1:1: remark: Function Name: _Z4kernv [-Rpass]\nx.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-R]\n"
                 "x.hip:1:1: remark:     VGPRs Spill: 0 [-R]\n")
    assert chk.check_resources(str(p), "kern") == []
    p.write_text("x.hip:1:1: remark: Function Name: _Z4kernv [-Rpass]\nx.hip:1:1: remark:     ScratchSize [bytes/lane]: 16 [-R]\n"
                 "x.hip:1:1: remark:     VGPRs Spill: 3 [-R]\n")
    assert len(chk.check_resources(str(p), "kern")) == 2
