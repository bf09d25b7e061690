"""Regression aimed at one class of bug: a hand-emitted MFMA that reads an operand register before the value meant
for it has arrived (an operand moved into place by the register allocator one instruction earlier, or a fragment of
the previous step still sitting there).  The library's static check of the generated assembly guards against it; this
is the dynamic counterpart for the builds in which such a move was once found or flagged: every dropout
instantiation of the forward, dQ and dK/dV kernels and every instantiation of the forward for head dims above 128.

Ordinary N(0,1) inputs spread a logit over all contraction steps, so one stale step moves it by a fraction of its
standard deviation and the outputs by little more than the tolerance.  Here every query and key carries its weight in
ONE 16-wide slice of the head dim (which slice depends on the row), so a logit comes from a single contraction step of
a single MFMA and is either large (slices match: standard deviation about 4, the softmax is dominated by a few keys) or
near zero; a stale operand in any step then turns a dominant key into a negligible one or the reverse and moves O and
the gradients by order one.  Everything is compared with the CPU oracle to the usual bar."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu
SEED = 0x2545F4914F6CDD1D


def _slice_dominated(tag, stream, B, H, S, D, amp):
    """[B,H,S,D] bf16 bits: N(0, 0.05^2) everywhere plus N(0, amp^2) in the 16-wide slice (7 s + 3 h + stream) mod (D/16)."""
    x = 0.05 * W.normal_f32(tag, stream, B * H * S * D).reshape(B, H, S, D)
    big = amp * W.normal_f32(tag, stream + 10, B * H * S * 16).reshape(B, H, S, 16)
    n_slices = D // 16
    for h in range(H):
        which = (7 * np.arange(S) + 3 * h) % n_slices
        for c in range(n_slices):
            rows = np.nonzero(which == c)[0]
            x[:, h, rows, 16 * c:16 * c + 16] += big[:, h, rows]
    return W.f32_to_bf16_bits(x.astype(np.float32))


def _case(tag, B, H, Sq, Sk, D):
    scale = 1.0 / math.sqrt(D)
    amp = math.sqrt(4.0 / (4.0 * scale))           # matching slices: logit std = 4 amp^2 scale = 4
    q = _slice_dominated(tag, 0, B, H, Sq, D, amp)
    k = _slice_dominated(tag, 1, B, H, Sk, D, amp)
    v = W.f32_to_bf16_bits(0.5 * W.normal_f32(tag, 2, B * H * Sk * D).reshape(B, H, Sk, D))
    do = W.f32_to_bf16_bits(0.5 * W.normal_f32(tag, 3, B * H * Sq * D).reshape(B, H, Sq, D))
    return q, k, v, do, scale


def test_the_inputs_do_what_the_test_needs(oracle):
    """One slice carries the logit: dropping the dominant slice of the queries changes O by order one."""
    q, k, v, _, scale = _case(7100, 1, 2, 96, 160, 128)
    o, _, o32 = oracle.sdpa_fwd(q, k, v, scale, want_f32=True)
    qf = oracle.bf16_to_f32(q).copy()
    for h in range(2):
        which = (7 * np.arange(96) + 3 * h) % 8
        for i in range(96):
            if which[i] == 2:
                qf[0, h, i, 32:48] = 0.0          # what one stale contraction step would do to these rows
    _, _, o32_stale = oracle.sdpa_fwd(W.f32_to_bf16_bits(qf), k, v, scale, want_f32=True)
    assert np.abs(o32 - o32_stale).max() > 0.3


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("with_mask", [False, True])
@pytest.mark.parametrize("causal", [False, True])
def test_dropout_builds_on_slice_dominated_logits(oracle, D, with_mask, causal):
    from flame_amd import capi
    B, H, Sq, Sk = 1, 2, 200, 328
    print(f"[operand hazards] dropout D={D} mask={with_mask} causal={causal}", flush=True)
    q, k, v, do, scale = _case(7200 + D, B, H, Sq, Sk, D)
    p = float(np.quantile(oracle.dropout_uniforms(B, H, Sq, Sk, SEED), 0.25))
    keep = None
    if with_mask:
        keep = (W.normal_f32(7300, 0, B * H * Sq * Sk).reshape(B, H, Sq, Sk) > -0.8).astype(np.uint8)
        keep[..., 0] = 1
    mask = None if keep is None else torch.from_numpy(keep).cuda()
    dq_, dk_, dv_, ddo = (to_dev(t) for t in (q, k, v, do))
    o, lse = capi.attn_fwd_dropout(dq_, dk_, dv_, scale, p, SEED, causal=causal, mask=mask)
    ro, rlse, ro32 = oracle.sdpa_fwd_dropout(q, k, v, scale, p, SEED, causal=causal, mask=keep, want_f32=True)
    # the backward on the oracle's O and log-sum-exp: identical inputs on both sides
    lse_ref = torch.from_numpy(rlse.reshape(B * H, Sq)).cuda()
    g = capi.attn_bwd_dropout(dq_, dk_, dv_, to_dev(ro), ddo, lse_ref, scale, p, SEED, causal=causal, mask=mask)
    torch.cuda.synchronize()
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    ref = oracle.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, SEED, causal=causal, mask=keep, want_f32=True)
    for i, (name, got) in enumerate((("dQ", g[0]), ("dK", g[1]), ("dV", g[2]))):
        assert_close_bf16(oracle, name, to_f32(got), ref[i], ref[i + 3])


@pytest.mark.parametrize("D", [192, 256, 320, 384, 448, 512])
@pytest.mark.parametrize("causal", [False, True])
def test_big_head_dim_builds_on_slice_dominated_logits(oracle, D, causal):
    """All three chunk counts of the forward for head dims above 128 (D <= 256, <= 384, <= 512), whole and padded
    last chunks, many key tiles, with the keys split over workgroups (caller workspace) and not."""
    from flame_amd import capi
    B, H, Sq, Sk = 1, 2, 150, 1100
    print(f"[operand hazards] big head dim D={D} causal={causal}", flush=True)
    q, k, v, _, scale = _case(7400 + D, B, H, Sq, Sk, D)
    ro, rlse, ro32 = oracle.sdpa_fwd(q, k, v, scale, causal=causal, want_f32=True)
    dq_, dk_, dv_ = (to_dev(t) for t in (q, k, v))
    need = capi.fwd_workspace_bytes(B, H, Sq, Sk, D)
    assert need > 0
    for ws_bytes in (None, need):
        ws = None if ws_bytes is None else torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        o, lse = capi.attn_fwd(dq_, dk_, dv_, scale, causal=causal, workspace=ws)
        torch.cuda.synchronize()
        assert_close_bf16(oracle, f"O (workspace {ws_bytes})", to_f32(o), ro, ro32)
        fin = np.isfinite(rlse)
        glse = lse.cpu().numpy().reshape(rlse.shape)
        assert np.array_equal(np.isfinite(glse), fin) and oracle.max_abs(glse[fin], rlse[fin]) <= TOL_LSE
