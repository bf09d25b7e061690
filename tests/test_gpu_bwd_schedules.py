"""The selectable launch schedules of the backward (FLAME_ATTN_BWD_SCHEDULE: a pass of its own for the per-query rows,
then dQ and dK/dV workgroups in one grid, or the two kernels one after the other) against the default schedule and
against the CPU oracle.  The variable is read at every call, so one process runs all three."""
import os

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _bwd(schedule, *args, **kw):
    from flame_amd import capi
    old = os.environ.get("FLAME_ATTN_BWD_SCHEDULE")
    if schedule == "default":
        os.environ.pop("FLAME_ATTN_BWD_SCHEDULE", None)
    else:
        os.environ["FLAME_ATTN_BWD_SCHEDULE"] = schedule
    try:
        g = capi.attn_bwd(*args, **kw)
        torch.cuda.synchronize()
        return g
    finally:
        if old is None:
            os.environ.pop("FLAME_ATTN_BWD_SCHEDULE", None)
        else:
            os.environ["FLAME_ATTN_BWD_SCHEDULE"] = old


@pytest.mark.parametrize("B,H,S,D", [(1, 32, 2048, 128),      # 256 workgroups of 256 queries, 512 key blocks: whole rounds
                                     (1, 36, 2304, 128),      # 324 / 648: a partial last round, cut key blocks
                                     (2, 20, 2048, 64)])      # head dim 64
def test_joint_and_rows_schedules_against_default_and_oracle(oracle, B, H, S, D):
    from flame_amd import capi
    print(f"[bwd schedules] {B}x{H} S={S} D={D}", flush=True)
    shapes = [(B, H, S, D)] * 4
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(1300 + D, i, int(np.prod(s))).reshape(s)) for i, s in enumerate(shapes))
    scale = 1.0 / np.sqrt(D)
    dq_, dk_, dv_, ddo = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd(dq_, dk_, dv_, scale)
    base = _bwd("default", dq_, dk_, dv_, o, ddo, lse, scale)
    hd = (B * H) // 2
    # the backward of head hd on the library's own O and log-sum-exp rows (identical inputs on both sides)
    o_bits = o.view(torch.int16).cpu().numpy().view(np.uint16)
    ref = oracle.sdpa_bwd(q, k, v, o_bits, do, scale, heads=(hd, hd + 1), want_f32=True)
    for schedule in ("joint", "rows"):
        capi.profiling_enable(True)
        g = _bwd(schedule, dq_, dk_, dv_, o, ddo, lse, scale)
        launches = {kind: n for kind, (_, n) in capi.profiling_read().items() if n}
        capi.profiling_enable(False)
        # the schedule asked for is the one that ran
        assert launches.get("bwd_rows") == 1, launches
        assert ("bwd_joint" in launches) == (schedule == "joint") and ("bwd_dq" in launches) == (schedule == "rows"), launches
        for name, a, b in zip(("dQ", "dK", "dV"), g, base):
            # same kernels, the per-query rows formed by another pass: a last-bit difference in delta at most
            assert oracle.rel_l2(to_f32(a), to_f32(b)) < 2e-3, (schedule, name)
            assert float((a.float() - b.float()).abs().max()) <= 2e-2, (schedule, name)
        for i, name in enumerate(("dQ", "dK", "dV")):
            got = to_f32(g[i]).reshape(B * H, S, D)[hd]
            assert_close_bf16(oracle, f"{name} ({schedule}, head {hd})", got, ref[i].reshape(B * H, S, D)[hd],
                              ref[i + 3].reshape(B * H, S, D)[hd])


def test_schedule_switch_is_ignored_where_it_does_not_apply(oracle):
    """Causal, ragged or small problems keep the default schedule whatever the variable says."""
    from flame_amd import capi
    B, H, S, D = 1, 2, 200, 64
    shapes = [(B, H, S, D)] * 4
    q, k, v, do = (to_dev(W.f32_to_bf16_bits(W.normal_f32(1400, i, int(np.prod(s))).reshape(s))) for i, s in enumerate(shapes))
    scale = 1.0 / np.sqrt(D)
    o, lse = capi.attn_fwd(q, k, v, scale, causal=True)
    base = _bwd("default", q, k, v, o, do, lse, scale, causal=True)
    for schedule in ("joint", "rows", "nonsense"):
        g = _bwd(schedule, q, k, v, o, do, lse, scale, causal=True)
        for a, b in zip(g, base):
            assert torch.equal(a, b), schedule
