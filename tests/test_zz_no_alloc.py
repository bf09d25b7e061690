"""The allocation-free backward entry point (flame_attn_bwd_bf16_noalloc) against flame_attn_bwd_bf16,
through the C ABI: two calls in a row on the same GPU, the second with a smaller input, so that the
fixed scratch still holds the first call's contents when the second one runs."""
import ctypes
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import to_dev

pytestmark = pytest.mark.gpu


def _problem(seed, B, H, Sq, Sk, D):
    return [to_dev(W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D)))
            for s, n in enumerate((Sq, Sk, Sk, Sq))]


def _both(capi, q, k, v, do, scale, **kw):
    o, lse = capi.attn_fwd(q, k, v, scale, **kw)
    want = capi.attn_bwd(q, k, v, o, do, lse, scale, **kw)
    grads = tuple(torch.full_like(t, float("nan")) for t in (q, k, v))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    got = capi.attn_bwd_noalloc(q, k, v, o, do, lse, scale, grads, **kw)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() == before          # torch's allocator was not touched either
    for name, a, b in zip(("dQ", "dK", "dV"), got, want):
        assert torch.equal(a, b), name                           # same kernels, same schedule: bit-identical
    return got


def test_noalloc_backward_matches_the_workspace_entry_point_twice_in_a_row():
    from flame_amd import capi
    # first call: 27 x 128-key blocks per head x 12 heads = 324 key blocks > 256 compute units, so the last round
    # is split and the partial-sum part of the scratch is used as well as the row part
    q, k, v, do = _problem(901, 1, 12, 3456, 3456, 128)
    print("[noalloc] call 1: B=1 H=12 S=3456 D=128", flush=True)
    _both(capi, q, k, v, do, 1.0 / math.sqrt(128))
    # second call, smaller and of another shape class: ragged sizes, causal, key lengths, D = 64
    q, k, v, do = _problem(902, 2, 3, 333, 517, 64)
    kvl = torch.tensor([517, 200], dtype=torch.int32, device="cuda")
    print("[noalloc] call 2: B=2 H=3 Sq=333 Sk=517 D=64 causal + key lengths", flush=True)
    _both(capi, q, k, v, do, 0.125, causal=True, kv_len=kvl)
    # and a larger one again
    q, k, v, do = _problem(903, 1, 4, 1024, 2048, 128)
    print("[noalloc] call 3: B=1 H=4 Sq=1024 Sk=2048 D=128", flush=True)
    _both(capi, q, k, v, do, 0.09)


def test_noalloc_backward_rejects_more_rows_than_its_scratch_holds():
    from flame_amd import capi
    f = capi.lib().flame_attn_bwd_noalloc_max_rows
    f.restype = ctypes.c_int
    max_rows = int(f())
    assert max_rows == 1 << 20
    # shapes only: the size check comes before any pointer is looked at
    q = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16, device="cuda")
    st = (ctypes.c_int64 * 4)(64 * 64, 64 * 64, 64, 1)
    p = ctypes.c_void_p(q.data_ptr())
    rc = capi.lib().flame_attn_bwd_bf16_noalloc(p, p, p, p, p, p, p, p, p, 2, 1, max_rows // 2 + 1, 64, 64,
                                                ctypes.c_float(0.125), st, st, st, st, st, st, st, st,
                                                *(ctypes.c_int64(0) for _ in range(9)), 0, None, None, None, None)
    assert rc == capi.ERR_TOO_LARGE
