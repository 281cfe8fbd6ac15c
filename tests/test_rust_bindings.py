"""The Rust FFI crate (bindings/turq-sys/src/lib.rs) cannot be compiled in this tree (no Rust toolchain), so its `extern "C"` block
is checked against include/turq.h mechanically: the same functions in the same order, the same number of arguments, and for every
argument and return value the same pointer depth, constness and integer / float width.  Constants are compared by value."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

C_BASE = {"int": "c_int", "void": "c_void", "char": "c_char", "size_t": "usize", "int64_t": "i64", "uint64_t": "u64", "uint32_t": "u32",
          "float": "f32", "double": "f64", "turq_ctx": "turq_ctx", "turq_weight": "turq_weight", "turq_gguf": "turq_gguf",
          "turq_graph": "turq_graph"}


def c_type_to_rust(decl, is_param):
    """'const turq_weight *const *weights' -> '*const *const turq_weight' (the parameter name dropped)"""
    decl = " ".join(decl.split())
    array = False
    if is_param:
        m = re.match(r"^(.*?)(\w+)\s*\[\d*\]$", decl)
        if m:
            decl, array = m.group(1).strip(), True
        else:
            decl = re.match(r"^(.*?)(\w+)$", decl).group(1).strip()
    toks = re.findall(r"const|\*|\w+", decl)
    i, const = 0, False
    if toks[i] == "const":
        const, i = True, i + 1
    ty = C_BASE[toks[i]]
    i += 1
    if i < len(toks) and toks[i] == "const":
        const, i = True, i + 1
    while i < len(toks):
        assert toks[i] == "*", decl
        i += 1
        ty = ("*const " if const else "*mut ") + ty
        const = False
        if i < len(toks) and toks[i] == "const":
            const, i = True, i + 1
    return ("*mut " + ty) if array else ty


def header_prototypes():
    h = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "turq.h")).read(), flags=re.S)
    out = []
    for ret, name, args in re.findall(r"^\s*((?:const\s+)?[a-z_0-9]+\s*\**)\s*(turq_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", h, flags=re.M | re.S):
        args = " ".join(args.split())
        params = [] if args == "void" else [c_type_to_rust(a, True) for a in args.split(",")]
        r = c_type_to_rust(ret, False)
        out.append((name, params, None if r == "c_void" else r))
    return out


def rust_externs():
    src = open(os.path.join(ROOT, "bindings", "turq-sys", "src", "lib.rs")).read()
    block = re.search(r'extern "C" \{(.*?)\n\}', src, flags=re.S).group(1)
    out = []
    for name, args, ret in re.findall(r"pub fn (turq_\w+)\((.*?)\)(?:\s*->\s*([^;]+))?;", block, flags=re.S):
        params = [a.split(":", 1)[1].strip() for a in args.split(",") if a.strip()]
        out.append((name, params, ret.strip() if ret else None))
    return out, src


def test_every_entry_point_is_declared_with_the_same_signature():
    c, (r, _) = header_prototypes(), rust_externs()
    assert len(c) >= 49
    assert [p[0] for p in r] == [p[0] for p in c]          # same functions, same order
    for (name, cp, cr), (_, rp, rr) in zip(c, r):
        assert rp == cp, (name, rp, cp)
        assert rr == cr, (name, rr, cr)


def test_constants_match_the_header():
    h = open(os.path.join(ROOT, "include", "turq.h")).read()
    _, src = rust_externs()
    c_consts = {}
    for body in re.findall(r"enum\s*\{(.*?)\}", h, flags=re.S):
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        for name, val in re.findall(r"(TURQ_\w+)\s*=\s*(\d+)", body):
            c_consts[name] = int(val)
    m = re.search(r"#define TURQ_NOALLOC_SCRATCH_BYTES \((\d+)u << (\d+)\)", h)
    c_consts["TURQ_NOALLOC_SCRATCH_BYTES"] = int(m.group(1)) << int(m.group(2))
    for name, val in re.findall(r"#define (TURQ_\w+) (0x[0-9A-Fa-f]+)\b", h):      # flag values
        c_consts[name] = int(val, 16)
    r_consts = {}
    for name, val in re.findall(r"pub const (TURQ_\w+): \w+ = ([^;]+);", src):
        r_consts[name] = eval(val, {})
    assert r_consts == c_consts


def test_the_safe_wrapper_calls_only_declared_functions():
    (r, _), used = rust_externs(), set()
    src = open(os.path.join(ROOT, "bindings", "tur-hip", "src", "lib.rs")).read()
    code = "\n".join(l for l in src.split("\n") if not l.lstrip().startswith("//"))
    used = set(re.findall(r"\b(turq_[a-z0-9_]+)\s*\(", code))
    declared = {p[0] for p in r}
    assert used and used <= declared, used - declared
    # and with the right number of arguments
    arity = {p[0]: len(p[1]) for p in r}
    for name, args in re.findall(r"\b(turq_[a-z0-9_]+)\s*\(((?:[^()]|\([^()]*\))*)\)", code):
        depth, n, cur = 0, 0, ""
        for ch in args:
            if ch in "([":
                depth += 1
            elif ch in ")]":
                depth -= 1
            if ch == "," and depth == 0:
                n += 1
                cur = ""
            else:
                cur += ch
        n += 1 if cur.strip() else 0
        assert n == arity[name], (name, n, arity[name])


# FFI functions that the safe wrapper does not call, each for a stated reason; everything else it declares it must use
NOT_WRAPPED = {
    # device-pointer plumbing: candle has no HIP tensor type yet, so the wrapper stages host tensors (TURQ_MEM_HOST)
    "turq_dev_alloc", "turq_dev_free", "turq_memcpy_h2d", "turq_memcpy_d2h", "turq_ctx_stream", "turq_qmatmul_noalloc",
    "turq_graph_begin", "turq_graph_end", "turq_graph_launch", "turq_graph_destroy", "turq_ctx_scratch_info",
    # measurement aids
    "turq_profile_begin", "turq_profile_end", "turq_read_yardstick", "turq_prefill_plan", "turq_prefill_plan_multi", "turq_tuning_describe", "turq_ctx_device_info", "turq_version",
    # host-side layout transforms and geometry used by tools, not by the model path
    "turq_tile_host", "turq_untile_host", "turq_tiled_nbytes", "turq_block_elems", "turq_block_bytes",
    # candle's own code keeps the metadata and the name table of the file; the embedding and the quantizers have no caller in
    # LinearX (src/models/layers/mod.rs builds its table through candle)
    "turq_gguf_tensor_count", "turq_gguf_tensor_name", "turq_gguf_meta_u64", "turq_gguf_meta_f64", "turq_gguf_meta_str",
    "turq_gguf_read_tensor", "turq_gguf_last_error", "turq_embedding_lookup", "turq_quantize_q8_0", "turq_quantize_q8_k",
}


def test_the_safe_wrapper_uses_every_function_it_binds_or_says_why_not():
    (r, _) = rust_externs()
    src = open(os.path.join(ROOT, "bindings", "tur-hip", "src", "lib.rs")).read()
    code = "\n".join(l for l in src.split("\n") if not l.lstrip().startswith("//"))
    used = set(re.findall(r"\b(turq_[a-z0-9_]+)\s*\(", code))
    declared = {p[0] for p in r}
    assert NOT_WRAPPED <= declared, NOT_WRAPPED - declared
    assert not (used & NOT_WRAPPED), used & NOT_WRAPPED
    assert declared - used == NOT_WRAPPED, sorted((declared - used) ^ NOT_WRAPPED)
