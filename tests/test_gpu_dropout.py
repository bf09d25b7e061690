"""Dropout of the attention probabilities inside the fused kernels, through the C ABI, against the CPU oracle: the
kept set is the reference's (one xorshift round of seed ^ flat element index, src/rng/mod.rs:14-24 drawn over the whole
[B*H, Sq, Sk] tensor by src/autograd_v4/ops/sdpa.rs:229-231), so O, dQ, dK and dV match the oracle to the usual bar,
and the log-sum-exp is that of the undropped softmax, bit for bit."""
import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, TOL_MAX_ABS, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu

SEED = 0x2545F4914F6CDD1D
# The bar is the one of every other test: relative L2 1e-2 and the flat max-abs 2e-2 (one bf16 step where |x| >= 4).
# The backward is checked twice.  On the oracle's own O and log-sum-exp (identical inputs on both sides) it is held to
# that bar without exception.  Chained behind the library's forward, its delta = rowsum(dO * O) is formed from an O
# that differs from the oracle's by a bf16 step in places (a legitimate difference of two roundings), and with
# dropout O is large where a row attends few keys: a step of 2^-6 in O, summed over the head dim, moves delta by
# several hundredths and the gradients of those rows with it.  There, at most a fraction STRAGGLERS of a tensor's
# elements may miss the max-abs bar, by less than a factor of two; their errors and magnitudes are printed.
DROPOUT_MAX_ABS = TOL_MAX_ABS
STRAGGLERS = 1e-4


def _allowed(t):
    return max(1, int(STRAGGLERS * t.numel()))


def _check_grads(oracle, tag, g, ref, strict):
    for i, (name, got) in enumerate((("dQ", g[0]), ("dK", g[1]), ("dV", g[2]))):
        assert_close_bf16(oracle, f"{name} ({tag})", to_f32(got), ref[i], ref[i + 3], max_abs=DROPOUT_MAX_ABS,
                          stragglers=0 if strict else _allowed(got))


def _inputs(tag, B, H, Sq, Sk, D):
    shapes = [(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D), (B, H, Sq, D)]
    return [W.f32_to_bf16_bits(W.normal_f32(tag, i, int(np.prod(s))).reshape(s)) for i, s in enumerate(shapes)]


@pytest.mark.parametrize("B,H,Sq,Sk,D,causal,kv_len,p", [
    (2, 3, 200, 328, 64, False, None, 0.1),
    (2, 2, 256, 256, 128, True, None, 0.3),
    (2, 2, 130, 77, 128, False, [77, 40], 0.5),
    (1, 3, 192, 320, 96, True, None, 0.2),          # head dim padded inside the kernels
    (1, 2, 1024, 1024, 128, False, None, 0.1),      # several query and key tiles per workgroup
])
def test_dropout_forward_and_backward_against_oracle(oracle, B, H, Sq, Sk, D, causal, kv_len, p):
    from flame_amd import capi
    print(f"[dropout] {B}x{H} Sq={Sq} Sk={Sk} D={D} causal={causal} kv_len={kv_len} p={p}", flush=True)
    q, k, v, do = _inputs(950 + D + Sq, B, H, Sq, Sk, D)
    scale = 1.0 / np.sqrt(D)
    # One xorshift round gives neighbouring indices nearly the same uniform, so on small tensors a fixed p keeps
    # nearly all or nearly nothing: p is placed at the quantile of this tensor's own uniforms instead, which drops
    # that fraction of the elements whatever the seed.
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED), p))
    kept = float(oracle.dropout_keep_mask(B, H, Sq, Sk, p, SEED).mean())
    print(f"      p = {p:.6f}, kept fraction {kept:.3f}", flush=True)
    assert 0.3 < kept < 0.95
    kvl_np = None if kv_len is None else np.array(kv_len, np.int32)
    kvl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    dq_, dk_, dv_, ddo = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd_dropout(dq_, dk_, dv_, scale, p, SEED, causal=causal, kv_len=kvl)
    o_plain, lse_plain = capi.attn_fwd(dq_, dk_, dv_, scale, causal=causal, kv_len=kvl)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, causal=causal, kv_len=kvl_np, want_f32=True)
    tol = DROPOUT_MAX_ABS
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32, max_abs=tol)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    assert torch.equal(lse, lse_plain) or float((lse - lse_plain).abs().max()) <= 1e-6      # the undropped softmax's
    assert not torch.equal(o, o_plain)
    ref = oracle.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, SEED, causal=causal, kv_len=kvl_np, want_f32=True)
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    g_same = capi.attn_bwd_dropout(dq_, dk_, dv_, to_dev(ro), ddo, lse_ref, scale, p, SEED, causal=causal, kv_len=kvl)
    g = capi.attn_bwd_dropout(dq_, dk_, dv_, o, ddo, lse, scale, p, SEED, causal=causal, kv_len=kvl)
    torch.cuda.synchronize()
    _check_grads(oracle, "on the oracle's O and LSE", g_same, ref, strict=True)
    _check_grads(oracle, "behind the library's forward", g, ref, strict=False)
    # the same against the oracle that rounds P f and dS to bf16 before the four products that take them, as the
    # kernels must
    with oracle.operand_rounding():
        ro_r, _, ro32_r = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, causal=causal, kv_len=kvl_np, want_f32=True)
        ref_r = oracle.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, SEED, causal=causal, kv_len=kvl_np, want_f32=True)
    assert_close_bf16(oracle, "O (operands rounded)", to_f32(o), ro_r, ro32_r, max_abs=tol)
    _check_grads(oracle, "operands rounded, on the oracle's O and LSE", g_same, ref_r, strict=True)
    # teeth: the plain forward, rescaled or not, is far from this oracle
    assert oracle.rel_l2(to_f32(o_plain), ro32) > 0.05 and oracle.rel_l2(to_f32(o_plain) / (1 - p), ro32) > 0.05


@pytest.mark.parametrize("B,H,Sq,Sk,D,causal,per_head", [(2, 3, 200, 328, 64, False, False), (2, 2, 192, 256, 128, True, True)])
def test_dropout_with_a_keep_mask(oracle, B, H, Sq, Sk, D, causal, per_head):
    """The general masked kernels with dropout: exclusions first, the draw on what is left, as the reference applies
    them (mask into the logits, src/autograd_v4/ops/sdpa.rs:216-222, dropout on the probabilities, :229-231)."""
    from flame_amd import capi
    print(f"[dropout+mask] {B}x{H} Sq={Sq} Sk={Sk} D={D} causal={causal} per_head={per_head}", flush=True)
    q, k, v, do = _inputs(970 + D, B, H, Sq, Sk, D)
    scale = 1.0 / np.sqrt(D)
    keep = (W.normal_f32(971, 0, B * (H if per_head else 1) * Sq * Sk).reshape(B, H if per_head else 1, Sq, Sk) > -0.4).astype(np.uint8)
    keep[..., 0] = 1
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED), 0.25))
    tol = DROPOUT_MAX_ABS
    mask = torch.from_numpy(keep).cuda()
    dq_, dk_, dv_, ddo = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd_dropout(dq_, dk_, dv_, scale, p, SEED, causal=causal, mask=mask)
    g = capi.attn_bwd_dropout(dq_, dk_, dv_, o, ddo, lse, scale, p, SEED, causal=causal, mask=mask)
    ro, rlse, ro32 = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, causal=causal, mask=keep, want_f32=True)
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    g_same = capi.attn_bwd_dropout(dq_, dk_, dv_, to_dev(ro), ddo, lse_ref, scale, p, SEED, causal=causal, mask=mask)
    torch.cuda.synchronize()
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32, max_abs=tol)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    ref = oracle.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, SEED, causal=causal, mask=keep, want_f32=True)
    _check_grads(oracle, "on the oracle's O and LSE", g_same, ref, strict=True)
    _check_grads(oracle, "behind the library's forward", g, ref, strict=False)


def test_dropout_kept_set_bit_exact_through_a_one_hot_value_matrix(oracle):
    """V = identity over the keys (Sk = D = 128) turns O into the dropped probabilities themselves: zero exactly
    where the reference's generator drops, non-zero elsewhere."""
    from flame_amd import capi
    B, H, Sq, Sk, D, p = 1, 2, 256, 128, 128, 0.4
    q, k, _, _ = _inputs(990, B, H, Sq, Sk, D)
    v = np.zeros((B, H, Sk, D), np.float32)
    v[..., np.arange(Sk), np.arange(D)] = 1.0
    vb = W.f32_to_bf16_bits(v)
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED), p))
    o, _ = capi.attn_fwd_dropout(to_dev(q), to_dev(k), to_dev(vb), 0.05, p, SEED)
    torch.cuda.synchronize()
    keep = oracle.dropout_keep_mask(B, H, Sq, Sk, p, SEED)
    got = to_f32(o)
    assert np.array_equal(got != 0, keep)
    assert 0.05 < keep.mean() < 0.95


@pytest.mark.parametrize("cq,ck", [(48, 40), (0, 33), (100, 0), (7, 128), (256, 128)])
def test_chunked_draw_kept_set_bit_exact(oracle, cq, ck):
    """The kept set of the reference's chunked configuration (one draw per chunk_q x chunk_kv tile, seeded per tile),
    read off O through a one-hot V; chunks that are not multiples of the kernels' tiles, along one axis only, and
    covering the whole tensor (the unchunked draw)."""
    from flame_amd import capi
    B, H, Sq, Sk, D = 1, 3, 256, 128, 128
    q, k, _, _ = _inputs(991, B, H, Sq, Sk, D)
    v = np.zeros((B, H, Sk, D), np.float32)
    v[..., np.arange(Sk), np.arange(D)] = 1.0
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED, cq, ck), 0.4))
    o, _ = capi.attn_fwd_dropout(to_dev(q), to_dev(k), to_dev(W.f32_to_bf16_bits(v)), 0.05, p, SEED, draw_chunk_q=cq, draw_chunk_kv=ck)
    torch.cuda.synchronize()
    keep = oracle.dropout_keep_mask(B, H, Sq, Sk, p, SEED, cq, ck)
    assert np.array_equal(to_f32(o) != 0, keep)
    assert 0.05 < keep.mean() < 0.95
    whole = (cq == 0 or cq >= Sq) and (ck == 0 or ck >= Sk)
    assert np.array_equal(keep, oracle.dropout_keep_mask(B, H, Sq, Sk, p, SEED)) == whole


@pytest.mark.parametrize("B,H,Sq,Sk,D,causal,cq,ck", [(2, 2, 200, 328, 64, False, 48, 100), (1, 2, 320, 256, 128, True, 130, 64)])
def test_chunked_draw_forward_and_backward_against_oracle(oracle, B, H, Sq, Sk, D, causal, cq, ck):
    from flame_amd import capi
    print(f"[dropout tiles] {B}x{H} Sq={Sq} Sk={Sk} D={D} causal={causal} tiles {cq} x {ck}", flush=True)
    q, k, v, do = _inputs(995 + D, B, H, Sq, Sk, D)
    scale = 1.0 / np.sqrt(D)
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED, cq, ck), 0.25))
    dq_, dk_, dv_, ddo = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd_dropout(dq_, dk_, dv_, scale, p, SEED, causal=causal, draw_chunk_q=cq, draw_chunk_kv=ck)
    g = capi.attn_bwd_dropout(dq_, dk_, dv_, o, ddo, lse, scale, p, SEED, causal=causal, draw_chunk_q=cq, draw_chunk_kv=ck)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, causal=causal, want_f32=True, chunk_q=cq, chunk_kv=ck)
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32, max_abs=DROPOUT_MAX_ABS)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    ref = oracle.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, SEED, causal=causal, want_f32=True, chunk_q=cq, chunk_kv=ck)
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    g_same = capi.attn_bwd_dropout(dq_, dk_, dv_, to_dev(ro), ddo, lse_ref, scale, p, SEED, causal=causal, draw_chunk_q=cq, draw_chunk_kv=ck)
    torch.cuda.synchronize()
    _check_grads(oracle, "on the oracle's O and LSE", g_same, ref, strict=True)
    _check_grads(oracle, "behind the library's forward", g, ref, strict=False)
    # teeth: the unchunked kept set gives another output
    ro_flat, _ = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, causal=causal)
    assert oracle.rel_l2(to_f32(o), oracle.bf16_to_f32(ro_flat)) > 0.05


def test_dropout_argument_checks():
    from flame_amd import capi
    q = torch.zeros((1, 1, 64, 64), dtype=torch.bfloat16, device="cuda")
    for bad in (-0.1, 1.0, 1.5, float("nan")):
        with pytest.raises(capi.FlameAttnError) as e:
            capi.attn_fwd_dropout(q, q, q, 0.125, bad, 1)
        assert e.value.code == capi.ERR_INVALID
    o, lse = capi.attn_fwd_dropout(q, q, q, 0.125, 0.0, 1)         # p = 0: the plain forward
    o2, lse2 = capi.attn_fwd(q, q, q, 0.125)
    torch.cuda.synchronize()
    assert torch.equal(o, o2) and torch.equal(lse, lse2)
