"""The launch-plan cache of flame_sdpa_chunked_bf16 on the GPU: a miss measures both query tiles and stores the
faster, the next call of the shape is a hit, masked problems have one tile and skip the measurement, a forced tile
and a cache file carried from one process to the next behave as the reference documents them
(cuda/src/flame_sdpa_stub.cu:1080-1379).  The output is checked against the oracle whichever tile runs.  The
environment is read once per process, so the cases that set it run in processes of their own."""
import ctypes
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import assert_close_bf16, to_dev, to_f32
from tests.test_plan_cache_file import FIELDS, ROOT

pytestmark = pytest.mark.gpu


class Stats(ctypes.Structure):
    _fields_ = [(f, ctypes.c_uint64) for f in FIELDS]


def _stats(lib):
    st = Stats()
    assert lib.flame_sdpa_autotune_get_stats(ctypes.byref(st)) == 0
    return {f: getattr(st, f) for f in FIELDS}


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _chunked(lib, q, k, v, out, scale, causal=0, mask=None, mask_heads=1):
    B, H, Q, D = q.shape
    K = k.shape[2]
    lib.flame_sdpa_chunked_bf16.restype = ctypes.c_int
    rc = lib.flame_sdpa_chunked_bf16(_p(q), _p(k), _p(v), B, H, Q, K, D, D, ctypes.c_float(scale), 64, causal, mask_heads,
                                     _p(mask), _p(out), None, ctypes.c_uint64(0),
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return rc


def test_miss_measures_hit_reuses_mask_skips(oracle):
    from flame_amd import capi
    lib = capi.lib()
    B, H, Q, K, D = 2, 5, 512, 320, 64
    print(f"[plan] {B}x{H} Q={Q} K={K} D={D}", flush=True)
    t = [W.f32_to_bf16_bits(W.normal_f32(911, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Q, K, K))]
    q, k, v = (to_dev(x) for x in t)
    out = torch.empty_like(q)
    ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, want_f32=True)
    lib.flame_sdpa_autotune_reset_stats()
    before = _stats(lib)
    assert _chunked(lib, q, k, v, out, 0.125) == 0
    assert_close_bf16(oracle, "O (first call)", to_f32(out), ro, ro32)
    s1 = _stats(lib)
    assert s1["cache_misses"] == 1 and s1["cache_hits"] == 0 and s1["tuned"] == 1 and s1["errors"] == 0
    assert s1["last_plan_source"] == 2 and s1["last_candidate_count"] == 2 and s1["last_best_time_ns"] > 0
    assert s1["last_q_chunk"] in (128, 256) and s1["last_k_chunk"] == 64
    assert s1["cache_entries"] == before["cache_entries"] + 1
    assert (s1["last_shape_b"], s1["last_shape_h"], s1["last_shape_q"], s1["last_shape_k"], s1["last_shape_dh"],
            s1["last_shape_dv"], s1["last_shape_mask_heads"], s1["last_shape_causal"]) == (B, H, Q, K, D, D, 0, 0)
    out.zero_()
    assert _chunked(lib, q, k, v, out, 0.125) == 0
    assert_close_bf16(oracle, "O (second call)", to_f32(out), ro, ro32)
    s2 = _stats(lib)
    assert s2["cache_hits"] == 1 and s2["cache_misses"] == 1 and s2["tuned"] == 1
    assert s2["last_plan_source"] == 1 and s2["last_q_chunk"] == s1["last_q_chunk"]
    # the causal flag is part of the key: another miss
    assert _chunked(lib, q, k, v, out, 0.125, causal=1) == 0
    roc, _, roc32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, causal=True, want_f32=True)
    assert_close_bf16(oracle, "O (causal)", to_f32(out), roc, roc32)
    s3 = _stats(lib)
    assert s3["cache_misses"] == 2 and s3["tuned"] == 2 and s3["last_shape_causal"] == 1
    # a mask leaves one tile: nothing to measure
    keep = (W.normal_f32(912, 0, B * Q * K).reshape(B, 1, Q, K) > -0.5).astype(np.uint8)
    keep[..., 0] = 1
    mask = torch.from_numpy(keep.astype(np.float32)).to(torch.bfloat16).cuda()
    assert _chunked(lib, q, k, v, out, 0.125, mask=mask, mask_heads=1) == 0
    rom, _, rom32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, mask=keep, want_f32=True)
    assert_close_bf16(oracle, "O (mask)", to_f32(out), rom, rom32)
    s4 = _stats(lib)
    assert s4["skipped"] == 1 and s4["tuned"] == 2 and s4["last_plan_source"] == 3 and s4["last_q_chunk"] == 128
    assert s4["last_shape_mask_heads"] == 1


CHILD = r"""
import ctypes, json, sys
sys.path.insert(0, %r)
import numpy as np, torch
from flame_amd import capi, workloads as W
from oracle import oracle as O
from tests.gpu_util import assert_close_bf16, to_dev, to_f32
from tests.test_gpu_plan_cache import _chunked, _stats
lib = capi.lib()
B, H, Q, K, D = 1, 4, 384, 256, 128
t = [W.f32_to_bf16_bits(W.normal_f32(913, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Q, K, K))]
q, k, v = (to_dev(x) for x in t)
out = torch.empty_like(q)
assert _chunked(lib, q, k, v, out, 0.09) == 0
ro, _, ro32 = O.sdpa_fwd(t[0], t[1], t[2], 0.09, want_f32=True)
assert_close_bf16(O, "O", to_f32(out), ro, ro32)
assert lib.flame_sdpa_autotune_flush_cache() == 0
print(json.dumps(_stats(lib)))
""" % ROOT


def _child(env_extra):
    env = {k: v for k, v in os.environ.items() if not k.startswith("FLAME_SDPA_")}
    env.update(env_extra)
    out = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert out.returncode == 0, out.stdout + out.stderr
    return json.loads(out.stdout.strip().splitlines()[-1])


@pytest.mark.parametrize("forced,ran,clamped", [("256", 256, 0), ("128", 128, 0), ("100", 128, 1), ("4096", 256, 1)])
def test_forced_tile(forced, ran, clamped):
    print(f"[plan] FLAME_SDPA_QCHUNK={forced}", flush=True)
    s = _child({"FLAME_SDPA_QCHUNK": forced})
    assert s["env_forced"] == 1 and s["clamped"] == clamped and s["last_plan_source"] == 4 and s["last_q_chunk"] == ran
    assert s["cache_hits"] == 0 and s["cache_misses"] == 0 and s["tuned"] == 0


def test_switched_off_takes_the_rule_and_counts_nothing():
    s = _child({"FLAME_SDPA_AUTOTUNE": "0"})
    assert s["cache_hits"] == 0 and s["cache_misses"] == 0 and s["tuned"] == 0 and s["cache_entries"] == 0
    assert s["last_plan_source"] == 3 and s["last_q_chunk"] == 128          # 12 workgroups of 128 rows: far from filling the chip


def test_cache_file_carries_a_plan_to_the_next_process(tmp_path):
    path = str(tmp_path / "sub" / "dir" / "plans.json")
    env = {"FLAME_SDPA_AUTOTUNE_CACHE": path, "FLAME_SDPA_AUTOTUNE_PERSIST": "1"}
    s1 = _child(env)
    assert s1["tuned"] == 1 and s1["cache_saved"] == 1 and s1["cache_entries"] == 1 and s1["last_plan_source"] == 2
    lines = open(path).read().splitlines()
    meta = json.loads(lines[0])["meta"]
    assert meta["version"] == 1 and meta["arch"].startswith("gfx950")
    entry = json.loads(lines[1])
    assert entry["key"] == {"B": 1, "H": 4, "Q": 384, "K": 256, "Dh": 128, "Dv": 128, "mask_heads": 0, "causal": 0}
    assert entry["plan"] == {"q": s1["last_q_chunk"], "k": 64}
    s2 = _child(env)
    assert s2["cache_loads"] == 1 and s2["cache_hits"] == 1 and s2["tuned"] == 0 and s2["last_plan_source"] == 1
    assert s2["last_q_chunk"] == s1["last_q_chunk"] and s2["cache_saved"] == 0      # nothing new to write
