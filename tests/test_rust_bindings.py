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
