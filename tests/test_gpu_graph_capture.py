"""The reference captures its backward into a CUDA graph and therefore requires the attention path to run without
allocation or host synchronisation in steady state (src/autograd.rs:1298-1311, src/cuda_graph.rs).  The native entry
points only enqueue kernels: here the forward and the backward (and the int8-QK forward with its quantisation) are
captured into a HIP graph through torch and replayed on new inputs, with eager work of the program's own between the
replays; every replay must reproduce the eager call bit for bit."""
import math

import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import to_dev

pytestmark = pytest.mark.gpu


def _rand(shape, seed, mul=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * mul).to(torch.bfloat16)


@pytest.mark.parametrize("B,H,Sq,Sk,D,causal", [(1, 24, 4608, 4608, 128, False), (2, 4, 320, 500, 64, True)])
def test_forward_and_backward_replay_from_a_graph(B, H, Sq, Sk, D, causal):
    from flame_amd import capi
    sc = 1.0 / math.sqrt(D)
    q, do = _rand((B, H, Sq, D), 1), _rand((B, H, Sq, D), 2)
    k, v = _rand((B, H, Sk, D), 3), _rand((B, H, Sk, D), 4)
    kvl = torch.tensor([Sk - 7 * b for b in range(B)], dtype=torch.int32, device="cuda") if causal else None
    ws = torch.empty(capi.bwd_workspace_bytes(B, H, Sq, D), dtype=torch.uint8, device="cuda")
    o = torch.empty_like(q)
    grads = tuple(torch.empty_like(t) for t in (q, k, v))

    def step(out, gr, w):
        _, lse = capi.attn_fwd(q, k, v, sc, causal=causal, kv_len=kvl, out=out)
        capi.attn_bwd(q, k, v, out, do, lse, sc, causal=causal, kv_len=kvl, workspace=w, grads=gr)
        return lse

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        step(o, grads, ws)                                  # first calls set kernel attributes: not inside a capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        lse_g = step(o, grads, ws)
    for rep in range(3):
        for t, seed in ((q, 10), (k, 11), (v, 12), (do, 13)):
            t.copy_(_rand(t.shape, seed + 10 * rep, mul=1.0 + 0.25 * rep))      # new inputs in the captured buffers
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in (o, lse_g, *grads)]
        # the same step eagerly, into other buffers, between the replays
        o2 = torch.empty_like(q)
        g2 = tuple(torch.empty_like(t) for t in (q, k, v))
        lse2 = step(o2, g2, torch.empty_like(ws))
        torch.cuda.synchronize()
        for name, a, b in zip(("O", "LSE", "dQ", "dK", "dV"), got, (o2, lse2, *g2)):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager call"


def test_int8_qk_forward_replays_from_a_graph():
    from flame_amd import capi
    B, H, S, D = 1, 8, 1024, 128
    q, k, v = _rand((B, H, S, D), 21), _rand((B, H, S, D), 22), _rand((B, H, S, D), 23)

    def step():
        qq = capi.sage_quant(q, k, smooth_k=True)
        return capi.sage_fwd(qq, v, 1.0 / math.sqrt(D))

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = step()
    o_g = out[0] if isinstance(out, tuple) else out
    for rep in range(3):
        for t, seed in ((q, 30), (k, 31), (v, 32)):
            t.copy_(_rand(t.shape, seed + 10 * rep))
        graph.replay()
        torch.cuda.synchronize()
        got = o_g.clone()
        ref = step()
        ref = ref[0] if isinstance(ref, tuple) else ref
        torch.cuda.synchronize()
        assert torch.equal(got, ref), f"replay {rep}"


_FIRST_CALL_SCRIPT = r'''
import math, sys
import torch
sys.path.insert(0, sys.argv[1])
from flame_amd import capi

B, H, S, D = 1, 1, 4096, 512
def rand(seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.randn((B, H, S, D), device="cuda", generator=g).to(torch.bfloat16)
q, k, v = rand(1), rand(2), rand(3)
need = capi.fwd_workspace_bytes(B, H, S, S, D)
assert need == 4 * S * (D + 1) * 4, need                 # 32 query tiles of 128: 4 slices of the keys each
ws = torch.empty(need, dtype=torch.uint8, device="cuda")
o = torch.empty_like(q)
lse = torch.empty(B * H, S, dtype=torch.float32, device="cuda")
sc = 1.0 / math.sqrt(D)
side = torch.cuda.Stream()
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph, stream=side):                # the first call into the library in this process
    capi.attn_fwd(q, k, v, sc, out=o, lse_out=lse, workspace=ws)
for rep in range(3):
    for t, seed in ((q, 10), (k, 11), (v, 12)):
        t.copy_(rand(seed + 10 * rep))
    graph.replay()
    torch.cuda.synchronize()
    got_o, got_lse = o.clone(), lse.clone()
    o2, lse2 = capi.attn_fwd(q, k, v, sc, workspace=torch.empty_like(ws))      # eager, other buffers
    o3, lse3 = capi.attn_fwd(q, k, v, sc)                                      # eager, unsplit
    torch.cuda.synchronize()
    assert torch.equal(got_o, o2) and torch.equal(got_lse, lse2), f"replay {rep} differs from the eager call"
    assert (got_o.float() - o3.float()).abs().max().item() <= 2e-2 and (got_lse - lse3).abs().max().item() <= 1e-3
print("CAPTURED_FIRST_CALL_OK")
'''


def test_key_split_forward_is_captured_on_its_first_call():
    """The forward for head dims above 128 on a small grid splits the keys over workgroups and needs room for partial
    outputs.  With the caller's workspace (flame_attn_fwd_ws_bf16) nothing is allocated, so even the first call of a
    process can be recorded into a graph: run in a process of its own, replayed on new inputs, bit-identical to the
    eager call and within tolerance of the unsplit forward."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("[graph capture] key-split forward (1,1,4096,512), first call of a fresh process", flush=True)
    res = subprocess.run([sys.executable, "-c", _FIRST_CALL_SCRIPT, root], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, timeout=110)
    assert res.returncode == 0 and "CAPTURED_FIRST_CALL_OK" in res.stdout, res.stdout[-3000:]
