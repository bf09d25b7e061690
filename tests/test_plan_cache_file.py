"""The launch-plan cache of the chunked entry point without a GPU: the counters' layout, and reading a cache file in
the reference's format (cuda/src/flame_sdpa_stub.cu:300-450).  The environment is read once per process, so each
case runs in a process of its own."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "flame_amd", "lib", "libflame_attn_hip.so")

FIELDS = ["env_forced", "clamped", "skipped", "fallback", "errors", "cache_hits", "cache_misses", "tuned", "last_q_chunk",
          "last_k_chunk", "cache_saved", "cache_loads", "cache_load_errors", "cache_entries", "last_candidate_count",
          "last_best_time_ns", "last_plan_source", "last_shape_b", "last_shape_h", "last_shape_q", "last_shape_k",
          "last_shape_dh", "last_shape_dv", "last_shape_mask_heads", "last_shape_causal"]

CHILD = r"""
import ctypes, json, sys
FIELDS = %r
class Stats(ctypes.Structure):
    _fields_ = [(f, ctypes.c_uint64) for f in FIELDS]
assert ctypes.sizeof(Stats) == 200
lib = ctypes.CDLL(%r)
st = Stats()
assert lib.flame_sdpa_autotune_get_stats(None) == 1      # the reference returns FLAME_CUDA_ERR_INVALID (cuda/src/flame_sdpa_stub.cu:1382-1385)
assert lib.flame_sdpa_autotune_get_stats(ctypes.byref(st)) == 0
first = {f: getattr(st, f) for f in FIELDS}
assert lib.flame_sdpa_autotune_flush_cache() == 0          # nothing changed: no file is written
assert lib.flame_sdpa_autotune_reset_stats() == 0
lib.flame_sdpa_autotune_get_stats(ctypes.byref(st))
print(json.dumps({"first": first, "after_reset": {f: getattr(st, f) for f in FIELDS}}))
""" % (FIELDS, LIB)


def _run(env_extra):
    env = {k: v for k, v in os.environ.items() if not k.startswith("FLAME_SDPA_")}
    env.update(env_extra)
    out = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    return json.loads(out.stdout.strip().splitlines()[-1])


def test_counters_start_at_zero_without_a_file():
    got = _run({})
    assert all(v == 0 for v in got["first"].values())


def test_cache_file_in_the_reference_format_is_read(tmp_path):
    f = tmp_path / "plans.json"
    f.write_text(
        '{"meta":{"version":1,"entries":3,"device":0,"sm":800,"driver":12000,"runtime":12000,"name":"x"}}\n'
        '{"key":{"B":1,"H":24,"Q":4608,"K":4608,"Dh":128,"Dv":128,"mask_heads":0,"causal":0},"plan":{"q":256,"k":64}}\n'
        '{ "key": { "B": 2, "H": 8, "Q": 512, "K": 512, "Dh": 64, "Dv": 64, "mask_heads": 1, "causal": 1 }, "plan": { "q": 128, "k": 64 } }\n'
        '# a comment\n'
        '4 16 1024 2049 64 64 0 0 128 64\n'
        'not a plan\n'
        '{"key":{"B":1,"H":1,"Q":1,"K":1,"Dh":64,"Dv":64,"mask_heads":0,"causal":0},"plan":{"q":0,"k":64}}\n')
    got = _run({"FLAME_SDPA_AUTOTUNE_CACHE": str(f), "FLAME_SDPA_AUTOTUNE_PERSIST": "1"})
    assert got["first"]["cache_entries"] == 3            # two JSON lines and the older ten-integer line
    assert got["first"]["cache_loads"] == 1
    assert got["first"]["cache_load_errors"] == 2        # the garbage line and the plan with q = 0
    assert got["first"]["cache_saved"] == 0
    assert got["after_reset"]["cache_loads"] == 0 and got["after_reset"]["cache_entries"] == 3
    assert not os.path.exists(str(f) + ".tmp")


def test_cache_file_of_another_version_is_ignored(tmp_path):
    f = tmp_path / "plans.json"
    f.write_text('{"meta":{"version":2}}\n'
                 '{"key":{"B":1,"H":24,"Q":4608,"K":4608,"Dh":128,"Dv":128,"mask_heads":0,"causal":0},"plan":{"q":256,"k":64}}\n')
    got = _run({"FLAME_SDPA_AUTOTUNE_CACHE": str(f), "FLAME_SDPA_AUTOTUNE_PERSIST": "1"})
    assert got["first"]["cache_entries"] == 0 and got["first"]["cache_load_errors"] == 1


def test_entry_limit_keeps_the_most_recent(tmp_path):
    f = tmp_path / "plans.json"
    lines = ['{"meta":{"version":1}}\n']
    for i in range(10):
        lines.append('{"key":{"B":%d,"H":1,"Q":256,"K":256,"Dh":64,"Dv":64,"mask_heads":0,"causal":0},"plan":{"q":128,"k":64}}\n' % (i + 1))
    f.write_text("".join(lines))
    got = _run({"FLAME_SDPA_AUTOTUNE_CACHE": str(f), "FLAME_SDPA_AUTOTUNE_PERSIST": "1", "FLAME_SDPA_AUTOTUNE_CACHE_LIMIT": "4"})
    assert got["first"]["cache_entries"] == 4
