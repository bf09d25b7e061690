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


_FORCED_128_SCRIPT = r"""
import sys
sys.path.insert(0, sys.argv[1])
import numpy as np, torch
from flame_amd import capi, workloads as W
B, H, S, D = 1, 32, 2048, 128
q, k, v, do = (torch.from_numpy(W.f32_to_bf16_bits(W.normal_f32(1500, i, B * H * S * D).reshape(B, H, S, D)).view(np.int16))
               .view(torch.bfloat16).cuda() for i in range(4))
scale = D ** -0.5
capi.profiling_enable(True)
o, lse = capi.attn_fwd(q, k, v, scale)
dq, dk, dv = capi.attn_bwd(q, k, v, o, do, lse, scale)
torch.cuda.synchronize()
torch.save({"o": o.cpu(), "lse": lse.cpu(), "dq": dq.cpu(), "dk": dk.cpu(), "dv": dv.cpu()}, sys.argv[2])
print("FORCED_128_DONE")
"""


def test_forced_128_query_workgroups_agree_with_the_256_query_ones(oracle, tmp_path):
    """FLAME_ATTN_WG_WAVES=4 (read once per process, hence a process of its own) makes the forward and dQ run their
    128-query kernels on a problem that would take the 256-query ones: same results to rounding, and head 7 against
    the oracle."""
    import subprocess
    import sys
    from flame_amd import capi
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "forced128.pt")
    env = dict(os.environ, FLAME_ATTN_WG_WAVES="4")
    print("[forced 128-query workgroups] 1x32 S=2048 D=128 in a process of its own", flush=True)
    res = subprocess.run([sys.executable, "-c", _FORCED_128_SCRIPT, root, out], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, timeout=110, env=env)
    assert res.returncode == 0 and "FORCED_128_DONE" in res.stdout, res.stdout[-3000:]
    forced = torch.load(out, weights_only=True)
    B, H, S, D = 1, 32, 2048, 128
    bits = [W.f32_to_bf16_bits(W.normal_f32(1500, i, B * H * S * D).reshape(B, H, S, D)) for i in range(4)]
    q, k, v, do = (to_dev(t) for t in bits)
    scale = D ** -0.5
    o, lse = capi.attn_fwd(q, k, v, scale)
    g = capi.attn_bwd(q, k, v, o, do, lse, scale)
    torch.cuda.synchronize()
    assert oracle.rel_l2(to_f32(forced["o"]), to_f32(o)) < 2e-3 and float((forced["lse"] - lse.cpu()).abs().max()) < 1e-4
    for name, a in zip(("dq", "dk", "dv"), g):
        assert oracle.rel_l2(to_f32(forced[name]), to_f32(a)) < 3e-3, name
    # other kernels did run there: the 128-query dQ kernel sums its key tiles in another order than the 256-query one
    assert not torch.equal(forced["dq"], g[0].cpu())
    hd = 7
    ro, rlse, ro32 = oracle.sdpa_fwd(bits[0], bits[1], bits[2], scale, heads=(hd, hd + 1), want_f32=True)
    assert_close_bf16(oracle, "O (forced 128)", to_f32(forced["o"])[0, hd], ro[0, hd], ro32[0, hd])
    ref = oracle.sdpa_bwd(bits[0], bits[1], bits[2], forced["o"].view(torch.int16).numpy().view(np.uint16), bits[3], scale,
                          heads=(hd, hd + 1), want_f32=True)
    for i, name in enumerate(("dq", "dk", "dv")):
        assert_close_bf16(oracle, f"{name} (forced 128)", to_f32(forced[name])[0, hd], ref[i][0, hd], ref[i + 3][0, hd])
