"""CPU-side checks of the drop-in boundary: the shared library loads (no GPU needed) and exports
every function that include/flame_attn.h declares; argument validation that needs no device work."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flame_attn.h")
LIB = os.path.join(ROOT, "flame_amd", "lib", "libflame_attn_hip.so")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(\w+)\s*\([^;{]*\)\s*;", text, flags=re.M)
    return sorted(set(n for n in names if n.startswith(("flame_", "sdpa_stream", "streaming_attn"))))


def _lib():
    if not os.path.exists(LIB):
        from flame_amd import build
        build.build_lib()
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_surface():
    names = _declared_functions()
    for must in ("flame_attn_fwd_bf16", "flame_attn_bwd_bf16", "flame_attn_bwd_workspace_bytes",
                 "flame_cudnn_sdpa_bf16", "flame_cudnn_sdpa_bf16_train_fwd", "flame_cudnn_sdpa_bwd_bf16",
                 "flame_flash_attention_bf16", "flame_sdpa_chunked_bf16", "streaming_attn_bf16_fp32_launch",
                 "sdpa_stream_bf16_launch", "flame_sage_quant_qk_int8", "flame_sage_attn_fwd_int8"):
        assert must in names, must


def test_library_exports_every_declared_symbol():
    lib = _lib()
    missing = [n for n in _declared_functions() if not hasattr(lib, n)]
    assert not missing, missing


def test_static_archive_defines_every_declared_symbol():
    """libflame_attn_hip.a is what a Rust build script links (the reference's build.rs links its kernels statically);
    it is made from the same object as the shared library."""
    import shutil
    import subprocess
    _lib()
    archive = os.path.join(os.path.dirname(LIB), "libflame_attn_hip.a")
    if not os.path.exists(archive):
        from flame_amd import build
        build.build_lib()
    if shutil.which("nm") is None:
        pytest.skip("nm not available")
    out = subprocess.run(["nm", "--defined-only", archive], stdout=subprocess.PIPE, text=True, check=True).stdout
    defined = {l.split()[-1] for l in out.splitlines() if len(l.split()) == 3 and l.split()[1] == "T"}
    missing = [n for n in _declared_functions() if n not in defined]
    assert not missing, missing


def test_argument_validation_without_a_device():
    lib = _lib()
    lib.flame_attn_bwd_workspace_bytes.restype = ctypes.c_size_t
    need = lib.flame_attn_bwd_workspace_bytes(1, 24, 4608, 128)
    rows = 2 * 24 * 4608 * 4                       # two fp32 rows per query: the required part
    slot = 2 * 128 * 128 * 4                       # fp32 dK/dV partials of one 128-key block
    assert need > rows and (need - rows) % slot == 0 and (need - rows) // slot >= 64
    assert lib.flame_attn_bwd_workspace_bytes(0, 1, 1, 64) == 0
    st = (ctypes.c_int64 * 4)(64 * 64, 64 * 64, 64, 1)
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)      # never dereferenced: validation fails first
    # non-positive sizes / scale -> -1, as the reference shim (src/cuda/cudnn_sdpa.cpp:326-328)
    assert lib.flame_attn_fwd_bf16(one, one, one, one, null, 0, 1, 64, 64, 64, ctypes.c_float(0.1), st, st, st, st,
                                   *(ctypes.c_int64(0),) * 5, 0, null, null, null, null) == -1
    assert lib.flame_attn_fwd_bf16(one, one, one, one, null, 1, 1, 64, 64, 64, ctypes.c_float(-1.0), st, st, st, st,
                                   *(ctypes.c_int64(0),) * 5, 0, null, null, null, null) == -1
    assert lib.flame_attn_fwd_bf16(null, one, one, one, null, 1, 1, 64, 64, 64, ctypes.c_float(0.1), st, st, st, st,
                                   *(ctypes.c_int64(0),) * 5, 0, null, null, null, null) == -1
    # head dims that are not a multiple of 8 or exceed 512, and a D stride of 2, are not built -> -2
    for bad_d in (100, 132, 520, 1024):
        assert lib.flame_attn_fwd_bf16(one, one, one, one, null, 1, 1, 64, 64, bad_d, ctypes.c_float(0.1), st, st, st, st,
                                       *(ctypes.c_int64(0),) * 5, 0, null, null, null, null) == -2
    bad = (ctypes.c_int64 * 4)(64 * 64, 64 * 64, 64, 2)
    assert lib.flame_attn_fwd_bf16(one, one, one, one, null, 1, 1, 64, 64, 64, ctypes.c_float(0.1), bad, st, st, st,
                                   *(ctypes.c_int64(0),) * 5, 0, null, null, null, null) == -2
    lib.flame_attn_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.flame_attn_version()


def test_product_package_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under flame_amd/ may reference it."""
    pkg = os.path.join(ROOT, "flame_amd")
    offenders = []
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                txt = open(os.path.join(d, f), errors="ignore").read()
                if re.search(r"\boracle\b", txt) and "import oracle" in txt or "from oracle" in txt or "liboracle" in txt:
                    offenders.append(os.path.join(d, f))
    assert not offenders, offenders
