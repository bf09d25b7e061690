"""Seeded sweep over shapes and option combinations: forward (O, LSE) and backward (dQ, dK, dV)
against the oracle through the C ABI.  Sizes straddle every loop threshold of the kernels (tiles of
64 keys / 64 and 128 queries, the pipelined steady-state loops that need several full tiles, ragged
tails, causal diagonals that cut tiles, per-batch key lengths including 0, explicit keep-masks with
fully excluded rows, [B,N,H,D]-strided views)."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    D = int(rng.choice([64, 128]))
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    Sq = int(rng.choice([1, 31, 64, 65, 127, 128, 129, 200, 257, 384, 450, 513]))
    Sk = int(rng.choice([1, 63, 64, 65, 128, 191, 192, 193, 256, 321, 448, 577, 640]))
    mode = ["none", "causal", "kvlen", "mask", "kvlen+causal"][seed % 5]
    strided = bool(rng.integers(0, 2))
    return rng, D, B, H, Sq, Sk, mode, strided


@pytest.mark.parametrize("seed", range(48))
def test_random_case(oracle, seed):
    from flame_amd import capi
    rng, D, B, H, Sq, Sk, mode, strided = _case(seed)
    print(f"[random] seed={seed} B={B} H={H} Sq={Sq} Sk={Sk} D={D} mode={mode} strided={strided}", flush=True)
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(5000 + seed, s, B * H * n * D).reshape(B, H, n, D))
                   for s, n in enumerate((Sq, Sk, Sk, Sq)))
    scale = 1.0 / math.sqrt(D)
    causal = "causal" in mode
    kv_len = mask = None
    if "kvlen" in mode:
        kv_len = rng.integers(0, Sk + 1, size=B).astype(np.int32)
        kv_len[0] = Sk if B > 1 else max(1, Sk - 3)
    if mode == "mask":
        mask = (rng.random((B, 1, Sq, Sk)) < 0.6).astype(np.uint8)
        mask[0, 0, Sq // 2] = 0                       # one fully excluded row

    def dev(bits):
        t = to_dev(bits)
        if strided:                                   # same values, memory laid out [B,N,H,D]
            t = t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        return t

    qd, kd, vd, dod = dev(q), dev(k), dev(v), dev(do)
    kvl = None if kv_len is None else torch.from_numpy(kv_len).cuda()
    md = None if mask is None else torch.from_numpy(mask).cuda()
    o, lse = capi.attn_fwd(qd, kd, vd, scale, causal=causal, kv_len=kvl, mask=md)
    dq, dk, dv = capi.attn_bwd(qd, kd, vd, o, dod, lse, scale, causal=causal, kv_len=kvl, mask=md)
    torch.cuda.synchronize()

    ro, rlse, rof = oracle.sdpa_fwd(q, k, v, scale, causal=causal, kv_len=kv_len, mask=mask, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o), ro, rof)
    got_lse = lse.cpu().numpy().reshape(rlse.shape)
    fin = np.isfinite(rlse)
    assert np.array_equal(np.isneginf(got_lse), np.isneginf(rlse))
    assert np.all(np.abs(got_lse[fin] - rlse[fin]) <= TOL_LSE)
    ref = oracle.sdpa_bwd(q, k, v, ro, do, scale, causal=causal, kv_len=kv_len, mask=mask, want_f32=True)
    for i, (name, got) in enumerate((("dQ", dq), ("dK", dk), ("dV", dv))):
        assert_close_bf16(oracle, name, to_f32(got), ref[i], ref[i + 3])
    if kv_len is not None:                            # keys past the length receive exactly zero gradient
        for b in range(B):
            assert not bool(dk[b, :, int(kv_len[b]):].any()) and not bool(dv[b, :, int(kv_len[b]):].any())


@pytest.mark.parametrize("seed", range(12))
def test_random_case_many_heads(oracle, seed):
    """Larger grids: enough workgroups that the kernels choose their 256-query workgroups and the dK/dV
    kernel splits its last scheduling round; oracle parity on the first and last (batch, head)."""
    from flame_amd import capi
    rng = np.random.default_rng(7000 + seed)
    D = int(rng.choice([64, 128]))
    B, H = int(rng.integers(1, 3)), int(rng.choice([12, 20, 33, 40]))
    Sq = int(rng.choice([512, 768, 1000, 1280, 1536]))
    Sk = int(rng.choice([512, 777, 1024, 1408]))
    mode = ["none", "causal", "kvlen", "none"][seed % 4]
    if mode == "causal":
        Sk = Sq
    print(f"[random many heads] seed={seed} B={B} H={H} Sq={Sq} Sk={Sk} D={D} mode={mode}", flush=True)
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(9000 + seed, s, B * H * n * D).reshape(B, H, n, D))
                   for s, n in enumerate((Sq, Sk, Sk, Sq)))
    scale = 1.0 / math.sqrt(D)
    causal = mode == "causal"
    kv_len = None
    if mode == "kvlen":
        kv_len = rng.integers(1, Sk + 1, size=B).astype(np.int32)
    kvl = None if kv_len is None else torch.from_numpy(kv_len).cuda()
    qd, kd, vd, dod = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd(qd, kd, vd, scale, causal=causal, kv_len=kvl)
    dq, dk, dv = capi.attn_bwd(qd, kd, vd, o, dod, lse, scale, causal=causal, kv_len=kvl)
    torch.cuda.synchronize()
    for hb in (0, B * H - 1):
        heads = (hb, hb + 1)
        ro, rlse, rof = oracle.sdpa_fwd(q, k, v, scale, causal=causal, kv_len=kv_len, heads=heads, want_f32=True)
        sel = lambda t, S: to_f32(t).reshape(B * H, S, D)[hb:hb + 1]
        assert_close_bf16(oracle, f"O[{hb}]", sel(o, Sq), ro.reshape(B * H, Sq, D)[hb:hb + 1], rof.reshape(B * H, Sq, D)[hb:hb + 1])
        assert np.max(np.abs(lse.cpu().numpy().reshape(B * H, Sq)[hb] - rlse.reshape(B * H, Sq)[hb])) <= TOL_LSE
        ref = oracle.sdpa_bwd(q, k, v, ro, do, scale, causal=causal, kv_len=kv_len, heads=heads, want_f32=True)
        for i, (name, got, S) in enumerate((("dQ", dq, Sq), ("dK", dk, Sk), ("dV", dv, Sk))):
            assert_close_bf16(oracle, f"{name}[{hb}]", sel(got, S), ref[i].reshape(B * H, S, D)[hb:hb + 1],
                              ref[i + 3].reshape(B * H, S, D)[hb:hb + 1])


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Sk", [64, 128, 192, 320, 448])
def test_wide_workgroups_short_key_walks(oracle, D, Sk):
    """256-query workgroups with 1, 2, 3, 5 and 7 key tiles: every way of entering and leaving the four-step
    pipeline of the forward and the three-stage walks of the backward, including copies clamped to the
    last tile."""
    from flame_amd import capi
    B, H, Sq = 1, 64, 1024
    print(f"[wide short walks] H={H} Sq={Sq} Sk={Sk} D={D}", flush=True)
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(31000 + Sk + D, s, B * H * n * D).reshape(B, H, n, D))
                   for s, n in enumerate((Sq, Sk, Sk, Sq)))
    scale = 1.0 / math.sqrt(D)
    qd, kd, vd, dod = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd(qd, kd, vd, scale)
    dq, dk, dv = capi.attn_bwd(qd, kd, vd, o, dod, lse, scale)
    torch.cuda.synchronize()
    for hb in (0, H - 1):
        heads = (hb, hb + 1)
        ro, rlse, rof = oracle.sdpa_fwd(q, k, v, scale, heads=heads, want_f32=True)
        sel = lambda t, S: to_f32(t).reshape(B * H, S, D)[hb:hb + 1]
        assert_close_bf16(oracle, f"O[{hb}]", sel(o, Sq), ro.reshape(B * H, Sq, D)[hb:hb + 1], rof.reshape(B * H, Sq, D)[hb:hb + 1])
        assert np.max(np.abs(lse.cpu().numpy().reshape(B * H, Sq)[hb] - rlse.reshape(B * H, Sq)[hb])) <= TOL_LSE
        ref = oracle.sdpa_bwd(q, k, v, ro, do, scale, heads=heads, want_f32=True)
        for i, (name, got, S) in enumerate((("dQ", dq, Sq), ("dK", dk, Sk), ("dV", dv, Sk))):
            assert_close_bf16(oracle, f"{name}[{hb}]", sel(got, S), ref[i].reshape(B * H, S, D)[hb:hb + 1],
                              ref[i + 3].reshape(B * H, S, D)[hb:hb + 1])
