"""Parsers for the two sides of the C ABI: the function declarations of include/flame_attn.h and the `extern "C"`
blocks of Rust source (rust/src/ffi.rs, the binding examples of the integration guide).  Used by the tests that hold the two
sides together; no GPU and no compiler needed."""
from __future__ import annotations

import re

# scalar / pointer types of the header -> the Rust spellings a binding may use for them
C_TO_RUST = {
    "void": {"()"},
    "int": {"c_int", "i32"},
    "float": {"f32", "c_float"},
    "bool": {"bool"},
    "long": {"c_long"},
    "size_t": {"usize"},
    "int64_t": {"i64"},
    "uint64_t": {"u64"},
    "const void*": {"*const c_void"},
    "void*": {"*mut c_void"},
    "const int64_t*": {"*const i64"},
    "const int32_t*": {"*const i32"},
    "const uint8_t*": {"*const u8"},
    "const float*": {"*const f32"},
    "float*": {"*mut f32"},
    "char*": {"*mut c_char"},
    "const char*": {"*const c_char"},
    "FlameAttnStatus": {"FlameAttnStatus", "c_int", "i32"},
    "FlameSdpaAutotuneStats*": {"*mut FlameSdpaAutotuneStats"},
    "FlameAttnKernelTimes*": {"*mut FlameAttnKernelTimes"},
}


def _strip_c_comments(text: str) -> str:
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _norm_c_type(t: str) -> str:
    t = re.sub(r"\s+", " ", t.strip())
    t = t.replace(" *", "*")
    return t


def parse_header(text: str) -> dict:
    """{function name: (return type, [(parameter type, parameter name), ...])} for every function declared in the
    header text (declarations end in ');', typedefs, enums and macros are skipped)."""
    text = _strip_c_comments(text)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)                  # preprocessor lines
    text = re.sub(r"typedef\s+(struct|enum)\b[^{;]*\{.*?\}[^;]*;", " ", text, flags=re.S)
    text = re.sub(r"\benum\s*\{.*?\}\s*;", " ", text, flags=re.S)
    text = re.sub(r'extern\s+"C"\s*\{', " ", text)
    out = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b([A-Za-z_]\w*)\s*\(([^()]*)\)\s*;", text):
        ret, name, params = _norm_c_type(m.group(1)), m.group(2), m.group(3).strip()
        plist = []
        if params and params != "void":
            for p in params.split(","):
                p = re.sub(r"\s+", " ", p.strip())
                pm = re.match(r"(.*?)([A-Za-z_]\w*)$", p)
                assert pm, f"cannot parse parameter {p!r} of {name}"
                plist.append((_norm_c_type(pm.group(1)), pm.group(2)))
        out[name] = (ret, plist)
    return out


def _norm_rust_type(t: str) -> str:
    t = re.sub(r"\s+", " ", t.strip())
    for prefix in ("core::ffi::", "std::ffi::", "std::os::raw::", "libc::"):
        t = t.replace(prefix, "")
    return t


def parse_rust_externs(text: str) -> dict:
    """{function name: (return type or "()", [(parameter name, parameter type), ...])} for every `fn` inside an
    `extern "C" { ... }` block of the text.  Declarations whose parameter list contains a comment (the abbreviated
    examples of a document) are returned with None for the parameters."""
    out = {}
    for block in re.finditer(r'extern\s+"C"\s*\{(.*?)\n\}', text, flags=re.S):
        body = block.group(1)
        for m in re.finditer(r"\bfn\s+([A-Za-z_]\w*)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", body, flags=re.S):
            name, params, ret = m.group(1), m.group(2), m.group(3)
            if "/*" in params:
                out[name] = (_norm_rust_type(ret or "()"), None)
                continue
            params = re.sub(r"//[^\n]*", " ", params)
            plist = []
            for p in params.split(","):
                p = p.strip()
                if not p:
                    continue
                pname, ptype = p.split(":", 1)
                plist.append((pname.strip(), _norm_rust_type(ptype)))
            out[name] = (_norm_rust_type(ret or "()"), plist)
    return out


def mismatches(c_decl, rust_decl) -> list:
    """Differences between one C declaration and its Rust counterpart: argument count, each argument's type, the
    return type.  Empty when they agree."""
    c_ret, c_params = c_decl
    r_ret, r_params = rust_decl
    problems = []
    if r_ret not in C_TO_RUST.get(c_ret, set()):
        problems.append(f"return type {r_ret!r} for C {c_ret!r}")
    if r_params is None:
        return problems
    if len(c_params) != len(r_params):
        problems.append(f"{len(r_params)} arguments for {len(c_params)} in the header")
        return problems
    for i, ((ctype, cname), (rname, rtype)) in enumerate(zip(c_params, r_params)):
        if rtype not in C_TO_RUST.get(ctype, set()):
            problems.append(f"argument {i} ({cname} / {rname}): {rtype!r} for C {ctype!r}")
    return problems
