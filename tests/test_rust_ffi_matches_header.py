"""The Rust side of the boundary cannot be compiled here (no Rust toolchain), so it is held to the C header by text:
every `extern "C"` declaration of rust/src/ffi.rs, and every one in the binding examples of the integration guide, must
name a function of include/flame_attn.h and agree with it in argument count and in every argument and return type;
and ffi.rs must declare every function the header has.  The calls in rust/src/sdpa.rs are checked for their
argument counts.  The same parsers then check that the shared library exports what the header declares."""
import os
import re

import pytest

from tests.capi_decls import mismatches, parse_header, parse_rust_externs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _read(*parts):
    with open(os.path.join(ROOT, *parts)) as f:
        return f.read()


@pytest.fixture(scope="module")
def header():
    decls = parse_header(_read("include", "flame_attn.h"))
    assert len(decls) >= 40 and "flame_attn_fwd_bf16" in decls and "flame_cudnn_sdpa_bwd_bf16" in decls
    return decls


def test_parsers_see_a_wrong_declaration(header):
    """Controls: a dropped argument, a wrong pointer constness, a wrong integer width and a wrong return type fail."""
    good = 'extern "C" {\n    pub fn flame_attn_bwd_workspace_bytes(b: c_int, h: c_int, n_q: c_int, d: c_int) -> usize;\n}'
    assert mismatches(header["flame_attn_bwd_workspace_bytes"], parse_rust_externs(good)["flame_attn_bwd_workspace_bytes"]) == []
    for bad in (good.replace("d: c_int", ""), good.replace("usize", "u32"), good.replace("h: c_int", "h: i64")):
        bad = bad.replace(", )", ")")
        assert mismatches(header["flame_attn_bwd_workspace_bytes"], parse_rust_externs(bad)["flame_attn_bwd_workspace_bytes"])
    fwd = parse_rust_externs(_read("rust", "src", "ffi.rs"))["flame_cudnn_sdpa_bf16"]
    swapped = (fwd[0], [(n, "*mut c_void" if t == "*const c_void" else t) for n, t in fwd[1]])
    assert mismatches(header["flame_cudnn_sdpa_bf16"], swapped)


def test_ffi_rs_declares_exactly_the_header(header):
    rust = parse_rust_externs(_read("rust", "src", "ffi.rs"))
    assert set(rust) == set(header), (sorted(set(header) - set(rust)), sorted(set(rust) - set(header)))
    for name, decl in rust.items():
        assert decl[1] is not None, f"{name}: abbreviated declaration in ffi.rs"
        assert mismatches(header[name], decl) == [], (name, mismatches(header[name], decl))
        names = [n for n, _ in decl[1]]
        assert len(set(names)) == len(names), f"{name}: duplicate parameter names {names}"


def test_ffi_rs_struct_layouts_match_the_header():
    """The two structs that cross the boundary: the same fields in the same order."""
    h, r = _read("include", "flame_attn.h"), _read("rust", "src", "ffi.rs")
    c_fields = re.search(r"typedef struct FlameSdpaAutotuneStats \{(.*?)\}", h, flags=re.S).group(1)
    c_names = [n.strip() for n in c_fields.replace("uint64_t", "").replace(";", "").split(",")]
    r_fields = re.search(r"pub struct FlameSdpaAutotuneStats \{(.*?)\}", r, flags=re.S).group(1)
    r_names = re.findall(r"pub (\w+): u64", r_fields)
    assert c_names == r_names and len(r_names) == 25
    kinds = int(re.search(r"FLAME_ATTN_N_KERNEL_KINDS = (\d+)", h).group(1))
    assert f"FLAME_ATTN_N_KERNEL_KINDS: usize = {kinds}" in r
    assert re.search(r"total_ms: \[f64; FLAME_ATTN_N_KERNEL_KINDS\],\s*pub launches: \[c_int; FLAME_ATTN_N_KERNEL_KINDS\]", r)
    for macro in ("FLAME_ATTN_ERR_INVALID", "FLAME_ATTN_ERR_UNSUPPORTED", "FLAME_ATTN_ERR_TOO_LARGE"):
        c_val = int(re.search(r"#define %s \((-?\d+)\)" % macro, h).group(1))
        assert f"{macro}: c_int = {c_val}" in r


def test_binding_examples_of_the_integration_guide_match_the_header(header):
    rust = parse_rust_externs(_read("INTEGRATION.md"))
    assert {"flame_cudnn_sdpa_bf16", "flame_cudnn_sdpa_bf16_train_fwd", "flame_cudnn_sdpa_bwd_bf16", "flame_attn_fwd_bf16"} <= set(rust)
    for name, decl in rust.items():
        assert name in header, f"the integration guide declares {name}, which the header does not have"
        assert mismatches(header[name], decl) == [], (name, mismatches(header[name], decl))


def test_wrapper_calls_pass_as_many_arguments_as_the_header_takes(header):
    """The wrapper modules under rust/src: every `ffi::name(...)` call has the declared number of arguments."""
    import glob
    import os
    files = sorted(f for f in glob.glob(os.path.join(ROOT, "rust", "src", "*.rs")) if os.path.basename(f) not in ("ffi.rs", "lib.rs"))
    assert {os.path.basename(f) for f in files} >= {"sdpa.rs", "attention.rs", "sage_attention.rs", "autograd_v4.rs"}
    for f in files:
        _check_calls(open(f).read(), header, os.path.basename(f))


def _check_calls(src, header, where):
    calls = list(re.finditer(r"ffi::(flame_\w+)\(", src))
    assert len(calls) >= 2, where
    for m in calls:
        depth, i = 1, m.end()
        while depth:
            depth += {"(": 1, ")": -1}.get(src[i], 0)
            i += 1
        args = src[m.end():i - 1]
        flat, depth, n = "", 0, 0
        for ch in args:
            depth += {"(": 1, ")": -1}.get(ch, 0)
            flat += ch if depth == 0 or ch != "," else ";"
        n = len([a for a in flat.split(",") if a.strip()])
        assert n == len(header[m.group(1)][1]), (where, m.group(1), n, len(header[m.group(1)][1]))


def test_build_rs_compiles_for_gfx950_with_the_flags_of_the_python_build():
    from flame_amd import build as fb
    src = _read("rust", "build.rs")
    for flag in fb.FLAGS:
        if flag in ("-shared",):
            continue
        assert f'"{flag}"' in src, f"build.rs lacks {flag}"
    assert "--offload-arch=gfx950" in src and "nvcc" not in src.replace("loops nvcc", "")
    assert "static=flame_attn_hip" in src and "dylib=amdhip64" in src
