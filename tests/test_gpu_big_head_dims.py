"""Head dims above 128 (up to 512), forward only: the reference's entry points take any head dim and serve these
through their materialised path (src/sdpa.rs:483-587, :788-961; the attention of a VAE mid block is one head of
D = 512 over the latent positions).  O and LSE against the CPU oracle: whole and padded chunks of 128, the plain
and the two-wavefronts-per-query-block forms (above 256), causal, key lengths, ragged tiles, the split of the keys
over workgroups on small grids, strided views, the reference-named entry points; the cases the kernel does not serve are refused, not computed some other way."""
import ctypes
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _case(seed, B, H, Sq, Sk, D, mul=1.0, vmul=None):
    muls = (mul, mul, mul if vmul is None else vmul)
    return [W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D) * np.float32(muls[s]))
            for s, n in enumerate((Sq, Sk, Sk))]


def _check(oracle, t, scale, causal=False, kv_len=None, tag=""):
    from flame_amd import capi
    B, H, Sq, D = t[0].shape
    Sk = t[1].shape[2]
    print(f"[big head dim] D={D} B={B} H={H} Sq={Sq} Sk={Sk} causal={causal} kv_len={kv_len} {tag}", flush=True)
    q, k, v = (to_dev(x) for x in t)
    kvl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    ro, rlse, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], scale, causal=causal, kv_len=kv_len, want_f32=True)
    # without a workspace (never split), then, where the library would split the keys over workgroups, with the
    # workspace it asks for and with half of it (fewer slices)
    need = capi.fwd_workspace_bytes(B, H, Sq, Sk, D)
    first = None
    for ws_bytes in (None, need, need // 2) if need else (None,):
        ws = None if ws_bytes is None else torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        o = torch.full_like(q, float("nan"))       # a skipped store, or one past the head dim, shows
        _, lse = capi.attn_fwd(q, k, v, scale, causal=causal, kv_len=kvl, out=o, workspace=ws)
        torch.cuda.synchronize()
        assert_close_bf16(oracle, f"O (workspace {ws_bytes})", to_f32(o), ro, ro32)
        assert oracle.cosine(to_f32(o), ro32) >= 0.9999
        glse, rl = lse.cpu().numpy().reshape(rlse.shape), rlse
        fin = np.isfinite(rl)
        assert np.array_equal(np.isfinite(glse), fin) and oracle.max_abs(glse[fin], rl[fin]) <= TOL_LSE
        first = first or (o, lse)
    return first


@pytest.mark.parametrize("D", [136, 192, 256, 264, 320, 384, 392, 448, 512])
def test_big_head_dims_plain_and_exclusions(oracle, D):
    t = _case(5000 + D, 2, 2, 150, 203, D)
    sc = 1.0 / math.sqrt(D)
    _check(oracle, t, sc)
    _check(oracle, t, sc, causal=True)
    _check(oracle, t, sc, kv_len=[203, 37])
    _check(oracle, t, sc, causal=True, kv_len=[120, 0])


@pytest.mark.parametrize("Sq,Sk", [(1, 1), (31, 33), (64, 32), (129, 64), (260, 700)])
@pytest.mark.parametrize("D", [256, 512])
def test_big_head_dims_tile_edges(oracle, D, Sq, Sk):
    t = _case(5100 + D + Sq, 1, 3, Sq, Sk, D, mul=1.5, vmul=1.0)
    _check(oracle, t, 1.0 / math.sqrt(D))
    if Sq > 1:
        _check(oracle, t, 1.0 / math.sqrt(D), causal=True)


@pytest.mark.parametrize("B,H,S,D", [(2, 8, 2048, 256), (1, 8, 2048, 384), (1, 8, 2048, 512)])
def test_more_query_blocks_than_compute_units(oracle, B, H, S, D):
    """At least 256 workgroups (128 queries each up to D = 256, 64 above), 64 key tiles per walk, causal: every
    compute unit walks, and the walks differ in length."""
    t = _case(5150 + D, B, H, S, S, D)
    _check(oracle, t, 1.0 / math.sqrt(D), causal=True)


def test_vae_mid_block_shape(oracle):
    """One head of D = 512 over a 48 x 48 latent (2304 positions), batch 2: more workgroups than the chip has CUs
    for one batch element is not needed for parity; large logits (Q and K of standard deviation 2: logits of
    standard deviation 4) exercise the running maximum across many tiles, with V left at unit scale so that the flat
    2e-2 bound on O means what it means in the other tests."""
    t = _case(5200, 2, 1, 2304, 2304, 512, mul=2.0, vmul=1.0)
    _check(oracle, t, 1.0 / math.sqrt(512))


@pytest.mark.parametrize("D", [256, 384, 512])
def test_key_slices_on_small_grids(oracle, D):
    """The library asks for a workspace here (the assertion below), so _check also runs the split forms.
    One query tile and 66 key tiles: 8 workgroups walk 9 key tiles each (the last one 3, ending in a ragged tile) and
    a second kernel merges their partial outputs.  With a key length of 300 most slices are empty, with 0 all of them
    (O = 0, LSE = -inf); causal, the 100 queries see at most 4 tiles, one per slice."""
    from flame_amd import capi
    assert capi.fwd_workspace_bytes(1, 1, 100, 2100, D) == 8 * 100 * (D + 1) * 4
    assert capi.fwd_workspace_bytes(1, 1, 100, 2100, 128) == 0 and capi.fwd_workspace_bytes(4, 64, 4096, 2100, D) == 0
    t = _case(5300 + D, 1, 1, 100, 2100, D, mul=1.5, vmul=1.0)
    sc = 1.0 / math.sqrt(D)
    _check(oracle, t, sc)
    _check(oracle, t, sc, kv_len=[300])
    _check(oracle, t, sc, kv_len=[0])
    _check(oracle, t, sc, causal=True)
    # two heads and three query tiles: slices of several (batch, head, query tile) workgroups side by side
    t = _case(5310 + D, 1, 2, 300, 1000, D)
    _check(oracle, t, sc)
    _check(oracle, t, sc, causal=True, kv_len=[777])


def test_strided_views_and_reference_named_entry_points(oracle):
    from flame_amd import capi
    lib = capi.lib()
    B, H, S, D = 1, 3, 200, 320
    t = _case(5300, B, H, S, S, D)
    q, k, v = (to_dev(x) for x in t)
    o, lse = _check(oracle, t, 1.0 / math.sqrt(D))

    def bnhd(x):
        return x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)

    o2 = bnhd(torch.empty_like(q))
    capi.attn_fwd(bnhd(q), bnhd(k), bnhd(v), 1.0 / math.sqrt(D), out=o2)
    torch.cuda.synchronize()
    assert torch.equal(o, o2)
    # the reference's [B*H, N, D] symbol (scale 1/sqrt(D))
    o3 = torch.full_like(q, float("nan"))
    lse3 = torch.empty(B * H, S, dtype=torch.float32, device="cuda")
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.flame_flash_attention_bf16(p(q), p(k), p(v), p(o3), p(lse3), B * H, S, S, D, s) == 0
    torch.cuda.synchronize()
    assert torch.equal(o, o3) and torch.equal(lse.reshape(-1), lse3.reshape(-1))


def test_what_the_big_head_dim_kernel_does_not_serve_is_refused():
    from flame_amd import capi
    B, H, S, D = 1, 1, 64, 256
    q = torch.zeros(B, H, S, D, dtype=torch.bfloat16, device="cuda")
    mask = torch.ones(B, H, S, S, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError):
        capi.attn_fwd(q, q, q, 0.1, mask=mask)
    with pytest.raises(RuntimeError):
        capi.attn_fwd_dropout(q, q, q, 0.1, 0.5, 1)
    lse = torch.zeros(B, H, S, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError):
        capi.attn_bwd(q, q, q, q, q, lse, 0.1)
    for bad in (520, 260, 1024):
        x = torch.zeros(B, H, S, bad, dtype=torch.bfloat16, device="cuda")
        with pytest.raises(RuntimeError):
            capi.attn_fwd(x, x, x, 0.1)
    torch.cuda.synchronize()
