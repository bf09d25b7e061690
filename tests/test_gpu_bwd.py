"""GPU parity of the tile-recompute backward (dQ, dK, dV) against the CPU oracle, through the C ABI."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _check_bwd(oracle, w, heads=None, tag=""):
    from flame_amd import capi
    print(f"[bwd] {w.name} {tag} shape={w.shape} causal={w.causal}", flush=True)
    q, k, v, do = (to_dev(t) for t in (w.q, w.k, w.v, w.do))
    kvl = None if w.kv_len is None else torch.from_numpy(w.kv_len).cuda()
    mask = None if w.mask is None else torch.from_numpy(w.mask).cuda()
    o, lse = capi.attn_fwd(q, k, v, w.scale, causal=w.causal, kv_len=kvl, mask=mask)
    dq, dk, dv = capi.attn_bwd(q, k, v, o, do, lse, w.scale, causal=w.causal, kv_len=kvl, mask=mask)
    torch.cuda.synchronize()
    B, H, Sq, Sk, D = w.shape
    # the oracle backward is fed the oracle's own bf16 O, not the kernel's
    ro, _ = oracle.sdpa_fwd(w.q, w.k, w.v, w.scale, causal=w.causal, kv_len=w.kv_len, mask=w.mask, heads=heads)
    ref = oracle.sdpa_bwd(w.q, w.k, w.v, ro, w.do, w.scale, causal=w.causal, kv_len=w.kv_len, mask=w.mask,
                          heads=heads, want_f32=True)
    hb, he = (0, B * H) if heads is None else heads
    for i, (name, got, S) in enumerate((("dQ", dq, Sq), ("dK", dk, Sk), ("dV", dv, Sk))):
        g = to_f32(got).reshape(B * H, S, D)[hb:he]
        assert_close_bf16(oracle, name, g, ref[i].reshape(B * H, S, D)[hb:he], ref[i + 3].reshape(B * H, S, D)[hb:he])
    return dq, dk, dv


def test_cfg1_small_noncausal(oracle):
    _check_bwd(oracle, W.config1())


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (37, 91), (64, 128), (129, 193), (300, 257)])
def test_partial_tiles(oracle, D, Sq, Sk):
    seed = 2000 + Sq * 7 + Sk
    B, H = 2, 2
    t = [W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D))
         for s, n in enumerate((Sq, Sk, Sk, Sq))]
    _check_bwd(oracle, W.Workload(f"partial_{Sq}x{Sk}_d{D}", t[0], t[1], t[2], t[3], 1.0 / math.sqrt(D)))


@pytest.mark.parametrize("D", [64, 128])
def test_causal(oracle, D):
    _check_bwd(oracle, W.config4(H=2, S=320, D=D))


def test_causal_rectangular(oracle):
    for Sq, Sk in ((100, 260), (260, 100)):
        t = [W.f32_to_bf16_bits(W.normal_f32(15 + Sq, s, 2 * n * 64).reshape(1, 2, n, 64))
             for s, n in enumerate((Sq, Sk, Sk, Sq))]
        _check_bwd(oracle, W.Workload(f"causal_rect_{Sq}x{Sk}", t[0], t[1], t[2], t[3], 0.125, causal=True))


def test_cfg3_ragged_key_lengths(oracle):
    w = W.config3(H=2, Sq=192)
    dq, dk, dv = _check_bwd(oracle, w)
    # gradients of padded keys are exactly zero
    for b, L in enumerate(w.kv_len):
        assert torch.all(dk[b, :, int(L):] == 0) and torch.all(dv[b, :, int(L):] == 0)


def test_general_keep_mask_and_fully_masked_rows(oracle):
    B, H, Sq, Sk, D = 2, 2, 70, 150, 64
    t = [W.f32_to_bf16_bits(W.normal_f32(87, s, B * H * n * D).reshape(B, H, n, D))
         for s, n in enumerate((Sq, Sk, Sk, Sq))]
    mask = (W.normal_f32(88, 0, B * H * Sq * Sk).reshape(B, H, Sq, Sk) > 0.3).astype(np.uint8)
    mask[0, 1, 5, :] = 0
    mask[:, :, :, 149] = 0          # a key nobody attends to: dK = dV = 0 there
    w = W.Workload("general_mask", t[0], t[1], t[2], t[3], 0.2, mask=mask)
    dq, dk, dv = _check_bwd(oracle, w)
    assert torch.all(dq[0, 1, 5] == 0)
    assert torch.all(dk[:, :, 149] == 0) and torch.all(dv[:, :, 149] == 0)


@pytest.mark.parametrize("D,Sq,Sk,mshape,with_len,causal", [
    (128, 192, 256, "full", False, False),      # a mask per (batch, head, query, key)
    (64, 128, 384, "full", True, False),        # ... together with per-batch key lengths
    (128, 128, 256, "keys", False, False),      # key padding mask [B,1,1,Sk], broadcast over heads and queries
    (64, 256, 128, "queries", False, False),    # [B,1,Sq,Sk]
    (128, 256, 256, "full", True, True),        # mask, key lengths and the causal flag together
])
def test_keep_mask_over_whole_tiles(oracle, D, Sq, Sk, mshape, with_len, causal):
    """Mask rows that are contiguous and 16-byte aligned, Sq a multiple of 64 and Sk of 128: the kernels that
    take the mask in 16-byte pieces (forward, dQ) and stage it through LDS (dK/dV)."""
    from flame_amd import capi
    B, H = 2, 3
    t = [W.f32_to_bf16_bits(W.normal_f32(311 + D, s, B * H * n * D).reshape(B, H, n, D))
         for s, n in enumerate((Sq, Sk, Sk, Sq))]
    rng = np.random.default_rng(Sq * 7 + Sk)
    shape = {"full": (B, H, Sq, Sk), "keys": (B, 1, 1, Sk), "queries": (B, 1, Sq, Sk)}[mshape]
    mask = (rng.random(shape) < 0.6).astype(np.uint8)
    mask[..., 0] = 1                                   # no row is emptied by accident ...
    if mshape != "keys":
        mask[0, 0, 5, :] = 0                           # ... one on purpose
    mask[..., Sk - 3] = 0                              # a key nobody attends to
    kv_len = np.asarray([Sk - 37, Sk], np.int32) if with_len else None
    w = W.Workload("mask_whole_tiles_" + mshape, t[0], t[1], t[2], t[3], 1.0 / math.sqrt(D), causal=causal,
                   kv_len=kv_len, mask=mask)
    dq, dk, dv = _check_bwd(oracle, w)
    if mshape != "keys":
        assert torch.all(dq[0, 0, 5] == 0)
    assert torch.all(dk[:, :, Sk - 3] == 0) and torch.all(dv[:, :, Sk - 3] == 0)
    if with_len:
        assert torch.all(dk[0, :, Sk - 37:] == 0) and torch.all(dv[0, :, Sk - 37:] == 0)
    # forward of the same problem
    q, k, v = (to_dev(x) for x in (w.q, w.k, w.v))
    kvl = None if kv_len is None else torch.from_numpy(kv_len).cuda()
    o, lse = capi.attn_fwd(q, k, v, w.scale, causal=causal, kv_len=kvl, mask=torch.from_numpy(mask).cuda())
    ro, rlse, rof = oracle.sdpa_fwd(w.q, w.k, w.v, w.scale, causal=causal, kv_len=kv_len, mask=mask, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o).reshape(B * H, Sq, D), ro.reshape(B * H, Sq, D), rof.reshape(B * H, Sq, D))
    glse = lse.cpu().numpy().reshape(B * H, Sq)
    fin = np.isfinite(rlse.reshape(B * H, Sq))
    assert np.array_equal(np.isfinite(glse), fin)
    assert np.max(np.abs(glse[fin] - rlse.reshape(B * H, Sq)[fin])) <= 1e-3


def test_strided_views_match_contiguous(oracle):
    from flame_amd import capi
    w = W.config2(H=3, n_text=40, grid=12, D=128)
    q, k, v, do = (to_dev(t) for t in (w.q, w.k, w.v, w.do))
    o, lse = capi.attn_fwd(q, k, v, w.scale)
    ref = capi.attn_bwd(q, k, v, o, do, lse, w.scale)

    def bnhd(t):   # same values, memory laid out [B,N,H,D]
        return t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)

    grads = tuple(bnhd(torch.empty_like(t)) for t in (q, k, v))
    got = capi.attn_bwd(bnhd(q), bnhd(k), bnhd(v), bnhd(o), bnhd(do), lse, w.scale, grads=grads)
    for a, b_ in zip(got, ref):
        assert torch.equal(a, b_)            # the layout changes no arithmetic: dQ, dK, dV bit-identical
    _check_bwd(oracle, w)


def test_cfg2_production_shape_head_subset(oracle):
    w = W.config2()
    _check_bwd(oracle, w, heads=(0, 1), tag="head 0")
    _check_bwd(oracle, w, heads=(23, 24), tag="head 23")


def test_workspace_too_small_is_rejected():
    from flame_amd import capi
    q = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16, device="cuda")
    o, lse = capi.attn_fwd(q, q, q, 0.125)
    ws = torch.empty(2 * 256 - 1, dtype=torch.uint8, device="cuda")     # the two fp32 rows per query need 2 x 256 B
    with pytest.raises(capi.FlameAttnError) as e:
        capi.attn_bwd(q, q, q, o, q, lse, 0.125, workspace=ws)
    assert e.value.code == capi.ERR_INVALID


def test_split_last_round_matches_unsplit_walk():
    """With the recommended workspace the key blocks of the last, partly filled scheduling round are
    split along the query walk and merged from fp32 partials; with the minimal workspace every block is
    walked by one workgroup.  Both orders of summation must agree to bf16 rounding, on every head."""
    from flame_amd import capi
    w = W.config2()
    B, H, Sq, Sk, D = w.shape
    q, k, v, do = (to_dev(t) for t in (w.q, w.k, w.v, w.do))
    o, lse = capi.attn_fwd(q, k, v, w.scale)
    rows_only = 2 * (-(-(B * H * Sq * 4) // 256) * 256)
    assert capi.bwd_workspace_bytes(B, H, Sq, D) > rows_only
    a = capi.attn_bwd(q, k, v, o, do, lse, w.scale)      # default workspace: split path for the last 96 key blocks
    b = capi.attn_bwd(q, k, v, o, do, lse, w.scale, workspace=torch.empty(rows_only, dtype=torch.uint8, device="cuda"))
    torch.cuda.synchronize()
    assert torch.equal(a[0], b[0])                       # dQ does not depend on the dK/dV schedule
    for name, x, y in (("dK", a[1], b[1]), ("dV", a[2], b[2])):
        xf, yf = x.float(), y.float()
        diff = (xf - yf).abs()
        ulp = torch.pow(2.0, torch.floor(torch.log2(yf.abs().clamp_min(2.0 ** -126))) - 7)
        assert bool((diff <= ulp + 1e-3).all()), (name, float(diff.max()))     # 1e-3: cancellation near zero
        whole = slice(0, 20)                             # heads whose key blocks all sit in the unsplit range
        assert torch.equal(x[:, whole], y[:, whole]), name


@pytest.mark.parametrize("mode", ["causal", "kvlen"])
def test_wide_workgroups_with_exclusions(oracle, mode):
    """Enough query tiles that the forward and dQ kernels pick their 256-query (8-wavefront)
    workgroups, combined with a causal diagonal or ragged key lengths; oracle parity on a head subset."""
    B, H, S, D = 2, 16, 2048, 128
    t = [W.f32_to_bf16_bits(W.normal_f32(4242, s, B * H * S * D).reshape(B, H, S, D) * np.float32(0.7071)) for s in range(4)]
    w = W.Workload(f"wide_{mode}", t[0], t[1], t[2], t[3], 1.0 / math.sqrt(D), causal=(mode == "causal"),
                   kv_len=np.array([S, 777], np.int32) if mode == "kvlen" else None)
    _check_bwd(oracle, w, heads=(0, 1), tag="first head")
    _check_bwd(oracle, w, heads=(B * H - 1, B * H), tag="last head")
