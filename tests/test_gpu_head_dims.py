"""Head dims other than the compiled 64 and 128: 96 (the third size of the reference's production path,
src/sdpa.rs:149, src/cuda/flash_attention_fwd.cu:307-324) and other multiples of 8 run zero-padded on the
next compiled size.  Forward and backward against the CPU oracle, plain and with every kind of exclusion,
on sizes that take each kernel variant (128- and 256-query workgroups, split dK/dV rounds)."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _case(seed, B, H, Sq, Sk, D, mul=1.0):
    return [W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D) * np.float32(mul))
            for s, n in enumerate((Sq, Sk, Sk, Sq))]


def _check(oracle, t, scale, causal=False, kv_len=None, mask=None, heads=None, tag=""):
    from flame_amd import capi
    B, H, Sq, D = t[0].shape
    Sk = t[1].shape[2]
    print(f"[head dim] D={D} B={B} H={H} Sq={Sq} Sk={Sk} causal={causal} kv_len={kv_len} mask={mask is not None} {tag}", flush=True)
    q, k, v, do = (to_dev(x) for x in t)
    kvl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    m = None if mask is None else torch.from_numpy(mask).cuda()
    # outputs start as NaN: a store that is skipped by mistake, or one past the head dim, shows
    o = torch.full_like(q, float("nan"))
    grads = tuple(torch.full_like(x, float("nan")) for x in (q, k, v))
    _, lse = capi.attn_fwd(q, k, v, scale, causal=causal, kv_len=kvl, mask=m, out=o)
    dq, dk, dv = capi.attn_bwd(q, k, v, o, do, lse, scale, causal=causal, kv_len=kvl, mask=m, grads=grads)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], scale, causal=causal, kv_len=kv_len, mask=mask, heads=heads,
                                     want_f32=True)
    ref = oracle.sdpa_bwd(t[0], t[1], t[2], ro, t[3], scale, causal=causal, kv_len=kv_len, mask=mask, heads=heads,
                          want_f32=True)
    hb, he = (0, B * H) if heads is None else heads

    def sel(x, S):
        return x.reshape(B * H, S, -1)[hb:he]

    assert_close_bf16(oracle, "O", sel(to_f32(o), Sq), sel(ro, Sq), sel(ro32, Sq))
    glse, rl = sel(lse.cpu().numpy(), Sq)[..., 0], sel(rlse, Sq)[..., 0]
    fin = np.isfinite(rl)
    assert np.array_equal(np.isfinite(glse), fin) and oracle.max_abs(glse[fin], rl[fin]) <= TOL_LSE
    for i, (name, g, S) in enumerate((("dQ", dq, Sq), ("dK", dk, Sk), ("dV", dv, Sk))):
        assert_close_bf16(oracle, name, sel(to_f32(g), S), sel(ref[i], S), sel(ref[i + 3], S))


@pytest.mark.parametrize("Sq,Sk", [(64, 64), (77, 203), (300, 257)])
def test_head_dim_96_plain_and_partial_tiles(oracle, Sq, Sk):
    _check(oracle, _case(960 + Sq, 2, 3, Sq, Sk, 96), 1.0 / math.sqrt(96))


def test_head_dim_96_reference_shapes(oracle):
    """N in {512}, 8 heads, HD = 96 (tests/fa2_parity_naive.rs:374-376 runs 64 and 128 there; 96 is the size its
    kernel also instantiates) through the reference-named symbol, and the training trio."""
    import ctypes
    from flame_amd import capi
    lib = capi.lib()
    BH, N, HD = 8, 512, 96
    t = _case(0xFA2 + HD, 1, BH, N, N, HD)
    q, k, v, do = (to_dev(x) for x in t)
    o = torch.empty_like(q)
    lse = torch.empty(BH, N, dtype=torch.float32, device="cuda")
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.flame_flash_attention_bf16(p(q), p(k), p(v), p(o), p(lse), BH, N, N, HD, s) == 0
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 1.0 / math.sqrt(HD), want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
    assert oracle.cosine(to_f32(o), ro32) >= 0.9999
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    dq, dk, dv = capi.cudnn_sdpa_bwd(q, k, v, o, do, lse, 1.0 / math.sqrt(HD))
    torch.cuda.synchronize()
    ref = oracle.sdpa_bwd(t[0], t[1], t[2], ro, t[3], 1.0 / math.sqrt(HD), want_f32=True)
    for i, (name, g) in enumerate((("dQ", dq), ("dK", dk), ("dV", dv))):
        assert_close_bf16(oracle, name, to_f32(g), ref[i], ref[i + 3])
        assert oracle.cosine(to_f32(g), ref[i + 3]) >= 0.9999


def test_head_dim_96_exclusions(oracle):
    t = _case(961, 2, 2, 200, 330, 96)
    sc = 1.0 / math.sqrt(96)
    _check(oracle, t, sc, causal=True)
    _check(oracle, t, sc, kv_len=[330, 91])
    mask = (W.normal_f32(962, 0, 2 * 2 * 200 * 330).reshape(2, 2, 200, 330) > 0.2).astype(np.uint8)
    mask[..., 0] = 1
    mask[1, 0, 7, :] = 0
    _check(oracle, t, sc, mask=mask)
    # whole tiles with vector-loadable mask rows: the lean masked kernels
    t = _case(963, 1, 3, 256, 384, 96)
    mask = (W.normal_f32(964, 0, 3 * 256 * 384).reshape(1, 3, 256, 384) > -0.3).astype(np.uint8)
    mask[..., 0] = 1
    _check(oracle, t, sc, mask=mask, causal=True, kv_len=[300])


@pytest.mark.parametrize("causal", [False, True])
def test_head_dim_96_wide_workgroups_and_split_rounds(oracle, causal):
    """Enough work for 256-query workgroups in the forward and dQ kernels and for a split last round in dK/dV."""
    B, H, S, D = 1, 12, 3456, 96
    t = _case(965, B, H, S, S, D, mul=0.8)
    for hd in (0, B * H - 1):
        _check(oracle, t, 1.0 / math.sqrt(D), causal=causal, heads=(hd, hd + 1), tag=f"head {hd}")


@pytest.mark.parametrize("D", [8, 32, 40, 72, 80, 112, 120])
def test_other_head_dims(oracle, D):
    t = _case(970 + D, 1, 2, 150, 190, D)
    _check(oracle, t, 1.0 / math.sqrt(D))
    _check(oracle, t, 1.0 / math.sqrt(D), causal=True, kv_len=[101])


def test_strided_views_with_head_dim_96(oracle):
    """The DiT layout: memory [B,N,H,D], passed as a [B,H,N,D] view (row stride H*96 elements)."""
    from flame_amd import capi
    B, H, S, D = 1, 4, 320, 96
    t = _case(981, B, H, S, S, D)
    q, k, v, do = (to_dev(x) for x in t)

    def bnhd(x):
        return x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)

    o, lse = capi.attn_fwd(q, k, v, 0.1)
    ref = capi.attn_bwd(q, k, v, o, do, lse, 0.1)
    o2 = bnhd(torch.empty_like(q))
    capi.attn_fwd(bnhd(q), bnhd(k), bnhd(v), 0.1, out=o2)
    grads = tuple(bnhd(torch.empty_like(x)) for x in (q, k, v))
    got = capi.attn_bwd(bnhd(q), bnhd(k), bnhd(v), o2, bnhd(do), lse, 0.1, grads=grads)
    torch.cuda.synchronize()
    assert torch.equal(o, o2)
    for a, b in zip(got, ref):
        assert torch.equal(a, b)
