"""The materialised path (flame_attn_fwd_materialised_bf16 / flame_attn_bwd_materialised_bf16): the shapes the fused
kernels refuse, which the reference serves through materialised scores as well (src/sdpa.rs:483-587, :788-961,
src/autograd.rs:801-848).  O, LSE, dQ, dK, dV against the CPU oracle to the usual bar: head dims that are not
multiples of 8, head dims above 128 with causal flag, key lengths, keep-mask and bias, head dims above 512, a value
head dim of its own, several bands of query rows against one, strided views, and agreement with the fused kernels
where both apply."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _case(tag, B, H, Sq, Sk, D, mul=1.0):
    shapes = [(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D), (B, H, Sq, D)]
    return [W.f32_to_bf16_bits(W.normal_f32(tag, i, int(np.prod(s))).reshape(s) * np.float32(mul if i < 2 else 1.0))
            for i, s in enumerate(shapes)]


def _check(oracle, t, scale, causal=False, kv_len=None, keep=None, ws_fwd=None, ws_bwd=None, tag=""):
    from flame_amd import capi
    q, k, v, do = t
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    print(f"[materialised] {B}x{H} Sq={Sq} Sk={Sk} D={D} causal={causal} kv_len={kv_len} mask={keep is not None} {tag}", flush=True)
    kvl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    kvl_np = None if kv_len is None else np.array(kv_len, np.int32)
    mask = None if keep is None else torch.from_numpy(keep).cuda()
    dq_, dk_, dv_, ddo = (to_dev(x) for x in t)
    o = torch.full_like(dq_, float("nan"))
    _, lse = capi.attn_fwd_materialised(dq_, dk_, dv_, scale, causal=causal, kv_len=kvl, mask=mask, out=o, workspace=ws_fwd)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd(q, k, v, scale, causal=causal, kv_len=kvl_np, mask=keep, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
    glse = lse.cpu().numpy().reshape(rlse.shape)
    fin = np.isfinite(rlse)
    assert np.array_equal(np.isfinite(glse), fin) and oracle.max_abs(glse[fin], rlse[fin]) <= TOL_LSE
    # the backward on the oracle's O and LSE: identical inputs on both sides
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    grads = tuple(torch.full_like(x, float("nan")) for x in (dq_, dk_, dv_))
    capi.attn_bwd_materialised(dq_, dk_, dv_, to_dev(ro), ddo, lse_ref, scale, causal=causal, kv_len=kvl, mask=mask, workspace=ws_bwd,
                               grads=grads)
    torch.cuda.synchronize()
    ref = oracle.sdpa_bwd(q, k, v, ro, do, scale, causal=causal, kv_len=kvl_np, mask=keep, want_f32=True)
    for i, (name, got) in enumerate((("dQ", grads[0]), ("dK", grads[1]), ("dV", grads[2]))):
        assert_close_bf16(oracle, name, to_f32(got), ref[i], ref[i + 3])
    return o, lse, grads


@pytest.mark.parametrize("D", [20, 52, 136, 256, 392, 520, 640])
def test_head_dims_the_fused_kernels_refuse(oracle, D):
    """Not a multiple of 8 (20, 52), above 128 (with exclusions and a backward), above 512."""
    B, H, Sq, Sk = 2, 2, 100, 150
    t = _case(8100 + D, B, H, Sq, Sk, D)
    sc = 1.0 / math.sqrt(D)
    _check(oracle, t, sc)
    _check(oracle, t, sc, causal=True)
    _check(oracle, t, sc, kv_len=[150, 37])
    keep = (W.normal_f32(8200 + D, 0, B * H * Sq * Sk).reshape(B, H, Sq, Sk) > -0.5).astype(np.uint8)
    keep[:, :, 3, :] = 0                      # a query row without an attended key: LSE = -inf, O = 0, zero gradients
    _check(oracle, t, sc, keep=keep)
    _check(oracle, t, sc, causal=True, kv_len=[120, 0], keep=keep)


def test_bias_and_broadcast_mask_at_head_dim_320(oracle):
    from flame_amd import capi
    B, H, Sq, Sk, D = 1, 3, 70, 90, 320
    q, k, v, _ = _case(8300, B, H, Sq, Sk, D)
    bias = (1.5 * W.normal_f32(8301, 0, H * Sq * Sk).reshape(1, H, Sq, Sk)).astype(np.float32)
    sc = 0.05
    o, lse = capi.attn_fwd_materialised(to_dev(q), to_dev(k), to_dev(v), sc, bias=torch.from_numpy(bias).cuda())
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd_bias(q, k, v, sc, bias, want_f32=True)
    assert_close_bf16(oracle, "O (bias)", to_f32(o), ro, ro32)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    # a key-padding mask broadcast over heads and queries, [B, 1, 1, Sk]
    keep = np.ones((B, 1, 1, Sk), np.uint8)
    keep[..., 60:] = 0
    t = _case(8302, B, H, Sq, Sk, D)
    _check(oracle, t, sc, keep=keep)


def test_value_head_dim_of_its_own(oracle):
    """Dv = 40 beside D = 72 (and Dv = 200 beside D = 136): the oracle has one head dim, so V and dO are zero-padded to
    D for it (padded columns change neither the softmax, nor delta, nor dP), or V is taken in column ranges."""
    from flame_amd import capi
    B, H, Sq, Sk, D, Dv = 1, 2, 120, 200, 72, 40
    q, k, v, do = _case(8400, B, H, Sq, Sk, D)
    v[..., Dv:] = 0
    do[..., Dv:] = 0
    sc = 1.0 / math.sqrt(D)
    qd, kd = to_dev(q), to_dev(k)
    vd, dod = to_dev(v)[..., :Dv].contiguous(), to_dev(do)[..., :Dv].contiguous()
    o, lse = capi.attn_fwd_materialised(qd, kd, vd, sc, causal=True)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd(q, k, v, sc, causal=True, want_f32=True)
    assert o.shape == (B, H, Sq, Dv)
    assert_close_bf16(oracle, "O", to_f32(o), ro[..., :Dv], ro32[..., :Dv])
    grads = (torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd))
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    capi.attn_bwd_materialised(qd, kd, vd, to_dev(ro)[..., :Dv].contiguous(), dod, lse_ref, sc, causal=True, grads=grads)
    torch.cuda.synchronize()
    ref = oracle.sdpa_bwd(q, k, v, ro, do, sc, causal=True, want_f32=True)
    assert_close_bf16(oracle, "dQ", to_f32(grads[0]), ref[0], ref[3])
    assert_close_bf16(oracle, "dK", to_f32(grads[1]), ref[1], ref[4])
    assert_close_bf16(oracle, "dV", to_f32(grads[2]), ref[2][..., :Dv], ref[5][..., :Dv])


def test_bands_of_query_rows(oracle):
    """A workspace that holds 48 and 32 query rows at a time (forward / backward): several bands, fp32 sums of dK and dV
    across them; the same bar, and close agreement with the one-band run."""
    from flame_amd import capi
    B, H, Sq, Sk, D = 2, 2, 200, 260, 264
    t = _case(8500, B, H, Sq, Sk, D)
    sc = 1.0 / math.sqrt(D)
    o1, lse1, g1 = _check(oracle, t, sc, causal=True, tag="one band")
    per_row_f, per_row_b = B * H * Sk * 6, B * H * Sk * 8
    rows_bytes = ((B * H * Sq * 4 + 255) // 256) * 256
    accum = ((B * H * Sk * 2 * D * 4 + 255) // 256) * 256
    ws_f = torch.empty(per_row_f * 48 + 1024, dtype=torch.uint8, device="cuda")
    ws_b = torch.empty(rows_bytes + accum + per_row_b * 32 + 1024, dtype=torch.uint8, device="cuda")
    o2, lse2, g2 = _check(oracle, t, sc, causal=True, ws_fwd=ws_f, ws_bwd=ws_b, tag="bands of 48 / 32 rows")
    # (not bit for bit: the GEMM library may sum a 48-row band in another order than a 200-row one)
    assert oracle.rel_l2(to_f32(o2), to_f32(o1)) < 2e-3 and float((lse1 - lse2).abs().max()) < 1e-4
    for a, b in zip(g1, g2):
        assert oracle.rel_l2(to_f32(b), to_f32(a)) < 3e-3
    # too little for 16 rows is refused, as is a missing workspace pointer
    small = torch.empty(per_row_f * 8, dtype=torch.uint8, device="cuda")
    with pytest.raises(capi.FlameAttnError) as e:
        capi.attn_fwd_materialised(*(to_dev(x) for x in t[:3]), sc, workspace=small)
    assert e.value.code == capi.ERR_INVALID
    assert capi.materialised_workspace_bytes(B, H, Sq, Sk, D, D, False) >= per_row_f * Sq
    assert capi.materialised_workspace_bytes(B, H, Sq, Sk, D, D, True) >= per_row_b * Sq + rows_bytes


def test_agrees_with_the_fused_kernels_and_takes_strided_views(oracle):
    from flame_amd import capi
    B, H, S, D = 2, 3, 256, 128
    t = _case(8600, B, H, S, S, D)
    sc = 1.0 / math.sqrt(D)
    o, lse, g = _check(oracle, t, sc, causal=True)
    q, k, v, do = (to_dev(x) for x in t)
    o_f, lse_f = capi.attn_fwd(q, k, v, sc, causal=True)
    g_f = capi.attn_bwd(q, k, v, o_f, do, lse_f, sc, causal=True)
    torch.cuda.synchronize()
    assert oracle.rel_l2(to_f32(o), to_f32(o_f)) < 5e-3 and float((lse.reshape(-1) - lse_f.reshape(-1)).abs().max()) < 1e-3
    for a, b in zip(g, g_f):
        assert oracle.rel_l2(to_f32(a), to_f32(b)) < 1e-2

    def bnhd(x):          # the [B,N,H,D] layout viewed as [B,H,N,D]
        return x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)

    o_s = bnhd(torch.empty_like(q))
    capi.attn_fwd_materialised(bnhd(q), bnhd(k), bnhd(v), sc, causal=True, out=o_s)
    torch.cuda.synchronize()
    assert oracle.rel_l2(to_f32(o_s), to_f32(o)) < 2e-3


def test_chunked_entry_point_of_the_reference_takes_any_head_dims(oracle):
    """flame_sdpa_chunked_bf16 (src/ffi/cuda_ffi.h:98-115) has no head-dim rule in the reference (scalar kernels,
    cuda/src/flame_sdpa_stub.cu:696-866): Dh = 264 with its bf16 keep-mask, and Dh = 36, run through the materialised
    path in the library's own scratch."""
    import ctypes
    from flame_amd import capi
    lib = capi.lib()
    lib.flame_sdpa_chunked_bf16.restype = ctypes.c_int
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for D, with_mask in ((264, True), (36, False)):
        B, H, Q, K = 2, 2, 70, 110
        q, k, v, _ = _case(8700 + D, B, H, Q, K, D)
        keep = None
        mask_bf16 = None
        if with_mask:
            keep = (W.normal_f32(8701, 0, B * Q * K).reshape(B, 1, Q, K) > -0.3).astype(np.uint8)
            keep[..., 0] = 1
            mask_bf16 = torch.from_numpy(keep.astype(np.float32)).to(torch.bfloat16).cuda()
        out = torch.full((B, H, Q, D), float("nan"), dtype=torch.bfloat16, device="cuda")
        qd, kd, vd = to_dev(q), to_dev(k), to_dev(v)
        rc = lib.flame_sdpa_chunked_bf16(p(qd), p(kd), p(vd), B, H, Q, K, D, D, ctypes.c_float(0.07), 64, 0, 1,
                                         p(mask_bf16) if with_mask else None, p(out), None, ctypes.c_uint64(0), stream)
        assert rc == 0
        torch.cuda.synchronize()
        ro, _, ro32 = oracle.sdpa_fwd(q, k, v, 0.07, mask=keep, want_f32=True)
        assert_close_bf16(oracle, f"O chunked entry point Dh={D}", to_f32(out), ro, ro32)


SEED = 0x2545F4914F6CDD1D


@pytest.mark.parametrize("B,H,Sq,Sk,D,causal,kv_len,with_mask,chunks,bands", [
    (2, 2, 200, 328, 136, False, None, False, (0, 0), False),
    (1, 3, 192, 256, 264, True, None, False, (0, 0), True),        # several bands of query rows
    (2, 2, 130, 77, 20, False, [77, 40], False, (0, 0), False),    # a head dim that is not a multiple of 8
    (1, 2, 160, 200, 320, False, None, True, (0, 0), False),       # keep-mask first, the draw on what is left
    (1, 2, 200, 328, 136, False, None, False, (64, 128), False),   # the kept set of the reference's chunked operator
])
def test_dropout_where_the_fused_kernels_refuse(oracle, B, H, Sq, Sk, D, causal, kv_len, with_mask, chunks, bands):
    """Dropout of the probabilities through the materialised path (head dims the fused dropout kernels do not take):
    the reference's kept set (src/rng/mod.rs:14-24 over the whole tensor, or tile by tile for its chunked operator),
    O, the log-sum-exp of the undropped softmax, and the backward on the oracle's own O and LSE, to the usual bar."""
    from flame_amd import capi
    print(f"[materialised dropout] {B}x{H} Sq={Sq} Sk={Sk} D={D} causal={causal} kv_len={kv_len} mask={with_mask} chunks={chunks} "
          f"bands={bands}", flush=True)
    q, k, v, do = _case(880 + D, B, H, Sq, Sk, D)
    scale = 1.0 / math.sqrt(D)
    cq, ck = chunks
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED, cq, ck), 0.3))
    kept = float(oracle.dropout_keep_mask(B, H, Sq, Sk, p, SEED, cq, ck).mean())
    assert 0.3 < kept < 0.95, kept
    keep = None
    if with_mask:
        keep = (W.normal_f32(881, 0, B * H * Sq * Sk).reshape(B, H, Sq, Sk) > -0.4).astype(np.uint8)
        keep[..., 0] = 1
    kvl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    kvl_np = None if kv_len is None else np.array(kv_len, np.int32)
    mask = None if keep is None else torch.from_numpy(keep).cuda()
    ws_f = ws_b = None
    if bands:          # room for 64 (forward) and 48 (backward) query rows per band, and the fp32 sums of dK and dV
        rows_bytes = ((B * H * Sq * 4 + 255) // 256) * 256
        accum = ((B * H * Sk * 2 * D * 4 + 255) // 256) * 256
        ws_f = torch.empty(B * H * Sk * 6 * 64 + 1024, dtype=torch.uint8, device="cuda")
        ws_b = torch.empty(rows_bytes + accum + B * H * Sk * 8 * 48 + 1024, dtype=torch.uint8, device="cuda")
    dq_, dk_, dv_, ddo = (to_dev(x) for x in (q, k, v, do))
    kw = dict(causal=causal, kv_len=kvl, mask=mask, dropout_p=p, dropout_seed=SEED, draw_chunk_q=cq, draw_chunk_kv=ck)
    o, lse = capi.attn_fwd_materialised(dq_, dk_, dv_, scale, workspace=ws_f, **kw)
    o_plain, lse_plain = capi.attn_fwd_materialised(dq_, dk_, dv_, scale, causal=causal, kv_len=kvl, mask=mask)
    torch.cuda.synchronize()
    okw = dict(causal=causal, kv_len=kvl_np, mask=keep, want_f32=True, chunk_q=cq, chunk_kv=ck)
    ro, rlse, ro32 = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, **okw)
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
    glse = lse.cpu().numpy().reshape(rlse.shape)
    fin = np.isfinite(rlse)
    assert np.array_equal(np.isfinite(glse), fin) and oracle.max_abs(glse[fin], rlse[fin]) <= TOL_LSE
    assert torch.equal(lse, lse_plain)                     # the undropped softmax's
    assert oracle.rel_l2(to_f32(o_plain), ro32) > 0.05     # teeth: the plain forward is far from this oracle
    # the kept set itself: O is zero in exactly ... cannot be read off O at these head dims; the backward, which draws
    # again, must agree with the oracle's on identical inputs
    ref = oracle.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, SEED, **okw)
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    g = capi.attn_bwd_materialised(dq_, dk_, dv_, to_dev(ro), ddo, lse_ref, scale, workspace=ws_b, **kw)
    torch.cuda.synchronize()
    for i, name in enumerate(("dQ", "dK", "dV")):
        assert_close_bf16(oracle, name, to_f32(g[i]), ref[i], ref[i + 3])


def test_dropout_kept_set_bit_exact_at_head_dim_136(oracle):
    """V = identity over the first 136 keys (Sk = 136 = Dv, head dim 136) turns O into the dropped probabilities
    themselves: zero exactly where the reference's generator drops, non-zero elsewhere."""
    from flame_amd import capi
    B, H, Sq, Sk, D = 1, 2, 64, 136, 136
    q, k, _, _ = _case(890, B, H, Sq, Sk, D, mul=0.25)          # small logits: every probability is far from zero
    v = np.zeros((B, H, Sk, D), np.float32)
    v[..., np.arange(Sk), np.arange(D)] = 1.0
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED), 0.4))
    o, _ = capi.attn_fwd_materialised(to_dev(q), to_dev(k), to_dev(W.f32_to_bf16_bits(v)), 1.0 / math.sqrt(D), dropout_p=p,
                                      dropout_seed=SEED)
    torch.cuda.synchronize()
    kept = oracle.dropout_keep_mask(B, H, Sq, Sk, p, SEED)
    assert np.array_equal(to_f32(o) != 0.0, kept)
