"""The Rust binding of the C ABI (rust/agpu-sys/src/lib.rs) against include/*.h: every declared function is bound,
nothing else is, and each binding has the header's arity, argument types and return type.  No Rust toolchain is
needed: both files are parsed as text.  The safe layer (rust/agpu-nn) may only call functions that are bound, with the
bound number of arguments."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SCALARS = {"int32_t": "i32", "uint32_t": "u32", "int64_t": "i64", "uint64_t": "u64", "size_t": "usize", "float": "f32",
           "char": "c_char", "void": "c_void"}


def c_type_to_rust(t):
    t = " ".join(t.split())
    const = t.startswith("const ")
    base = t[6:] if const else t
    stars = base.count("*")
    base = base.replace("*", "").strip()
    rust = SCALARS.get(base, base)
    if stars == 0:
        return "()" if base == "void" else rust
    out = rust
    for i in range(stars):
        out = ("*const " if (const and i == 0) else "*mut ") + out
    return out


def c_functions():
    fns = {}
    for fn in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if not fn.endswith(".h"):
            continue
        text = open(os.path.join(ROOT, "include", fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
        for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b(agpu_\w+)\s*\(([^)]*)\)\s*;", text):
            ret, name, params = " ".join(m.group(1).split()), m.group(2), m.group(3).strip()
            if "typedef" in ret:
                continue
            args = []
            if params and params != "void":
                for p in params.split(","):
                    p = " ".join(p.split())
                    args.append(c_type_to_rust(re.match(r"(.*?)(\w+)$", p).group(1).strip()))
            fns[name] = (c_type_to_rust(ret), args)
    return fns


def rust_functions():
    text = open(os.path.join(ROOT, "rust", "agpu-sys", "src", "lib.rs")).read()
    block = re.search(r'extern "C" \{(.*)\}', text, flags=re.S).group(1)
    block = re.sub(r"//.*$", "", block, flags=re.M)
    fns = {}
    for m in re.finditer(r"pub fn (agpu_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block):
        name, params, ret = m.group(1), m.group(2).strip(), (m.group(3) or "()").strip()
        args = [" ".join(p.split(":", 1)[1].split()) for p in params.split(",") if p.strip()] if params else []
        fns[name] = (" ".join(ret.split()), args)
    return fns


def test_every_header_function_is_bound_with_the_same_signature():
    c, r = c_functions(), rust_functions()
    assert len(c) >= 60
    assert set(c) == set(r), f"only in the headers: {sorted(set(c) - set(r))}; only in the binding: {sorted(set(r) - set(c))}"
    for name in sorted(c):
        assert c[name] == r[name], f"{name}: header {c[name]} != binding {r[name]}"


def test_config_struct_fields_match():
    header = open(os.path.join(ROOT, "include", "agpu_gpt2.h")).read()
    body = re.search(r"typedef struct agpu_gpt2_config \{(.*?)\} agpu_gpt2_config;", header, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    c_fields = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        ty, names = decl.split(" ", 1)
        c_fields += [(n.strip(), SCALARS[ty]) for n in names.split(",")]
    rust = open(os.path.join(ROOT, "rust", "agpu-sys", "src", "lib.rs")).read()
    rbody = re.search(r"pub struct agpu_gpt2_config \{(.*?)\}", rust, flags=re.S).group(1)
    r_fields = [(m.group(1), m.group(2)) for m in re.finditer(r"pub (\w+): (\w+),", rbody)]
    assert c_fields == r_fields


def test_constants_match_the_headers():
    rust = open(os.path.join(ROOT, "rust", "agpu-sys", "src", "lib.rs")).read()
    consts = {m.group(1): int(m.group(2), 0) for m in re.finditer(r"pub const (AGPU_\w+): \w+ = (-?(?:0x)?[0-9a-fA-F]+);", rust)}
    assert len(consts) >= 25
    for fn in ("agpu.h", "agpu_gpt2.h"):
        text = open(os.path.join(ROOT, "include", fn)).read()
        for m in re.finditer(r"#define (AGPU_\w+) \(?(-?(?:0x)?[0-9a-fA-F]+)u?\)?", text):
            name, value = m.group(1), int(m.group(2), 0)
            if name in ("AGPU_H", "AGPU_GPT2_H"):
                continue
            assert name in consts, f"{name} of {fn} has no Rust constant"
            assert consts[name] == value, name


def test_safe_layer_calls_only_bound_functions_with_the_bound_arity():
    bound = rust_functions()
    src_dir = os.path.join(ROOT, "rust", "agpu-nn", "src")
    calls = 0
    for fn in sorted(os.listdir(src_dir)):
        text = open(os.path.join(src_dir, fn)).read()
        for m in re.finditer(r"sys::(agpu_\w+)\s*\(", text):
            name = m.group(1)
            assert name in bound, f"{fn} calls {name}, which the binding does not declare"
            depth, i, n_args, any_arg = 1, m.end(), 0, False
            while depth:
                ch = text[i]
                if ch in "([{":
                    depth += 1
                elif ch in ")]}":
                    depth -= 1
                elif ch == "," and depth == 1:
                    n_args += 1
                if depth and not ch.isspace():
                    any_arg = True
                i += 1
            n_args = n_args + 1 if any_arg else 0
            assert n_args == len(bound[name][1]), f"{fn}: {name} called with {n_args} arguments, bound with {len(bound[name][1])}"
            calls += 1
    assert calls >= 40
