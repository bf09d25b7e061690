"""The ragged and the long causal configurations at their full sizes, through the C ABI.

Ragged cross attention (B=4, H=16, Sq=1024, Sk in {77, 333, 1024, 2049}, D=64) is small enough for the
CPU oracle to check every head (reference regression shapes: tests/sdpa_ragged_sk.rs:126-163).

Long causal self-attention (B=1, H=32, S=16384, D=128) costs the oracle 15 TFLOP in full, so it is
checked (a) against the oracle on three 128-row bands (first, middle, last) of the first and the last
head, where a band costs rows x S; dK and dV on the last 128 keys, which only the last band attends to;
(b) on all 32 heads through identities that hold at any size: sum_j dV_j = sum_i dO_i (the rows of P
sum to one) and sum_j dK_j ~ 0 (the rows of dS sum to zero); and (c) by the memory bound the path
exists for: nothing beyond the tensors of the problem and the declared workspace is ever allocated
(the reference's own long case is the ignored N=16384 test in tests/fa2_parity_naive.rs:391-418).
"""
import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def test_cfg3_ragged_cross_attention_full_size(oracle):
    from flame_amd import capi
    w = W.config3()
    B, H, Sq, Sk, D = w.shape
    assert (B, H, Sq, Sk, D) == (4, 16, 1024, 2049, 64)
    print(f"[full] {w.name} shape={w.shape} kv_len={w.kv_len.tolist()}", flush=True)
    q, k, v, do = (to_dev(t) for t in (w.q, w.k, w.v, w.do))
    kvl = torch.from_numpy(w.kv_len).cuda()
    o, lse = capi.attn_fwd(q, k, v, w.scale, kv_len=kvl)
    dq, dk, dv = capi.attn_bwd(q, k, v, o, do, lse, w.scale, kv_len=kvl)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sdpa_fwd(w.q, w.k, w.v, w.scale, kv_len=w.kv_len, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
    ml = oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse)
    print(f"      LSE max_abs={ml:.3e}", flush=True)
    assert ml <= TOL_LSE
    ref = oracle.sdpa_bwd(w.q, w.k, w.v, ro, w.do, w.scale, kv_len=w.kv_len, want_f32=True)
    for i, (name, got) in enumerate((("dQ", dq), ("dK", dk), ("dV", dv))):
        assert_close_bf16(oracle, name, to_f32(got), ref[i], ref[i + 3])
    for b, L in enumerate(w.kv_len):      # the padded keys hold +-1e4 and must not leak: exact zeros
        assert torch.all(dk[b, :, int(L):] == 0) and torch.all(dv[b, :, int(L):] == 0)
    # the same exclusions as a [B,1,1,Sk] keep-mask (the way the reference expresses them)
    mask = torch.from_numpy(w.extra["keep_mask"]).cuda()
    o2, lse2 = capi.attn_fwd(q, k, v, w.scale, mask=mask)
    g2 = capi.attn_bwd(q, k, v, o2, do, lse2, w.scale, mask=mask)
    torch.cuda.synchronize()
    assert_close_bf16(oracle, "O (keep-mask)", to_f32(o2), ro, ro32)
    for i, (name, got) in enumerate((("dQ (keep-mask)", g2[0]), ("dK (keep-mask)", g2[1]), ("dV (keep-mask)", g2[2]))):
        assert_close_bf16(oracle, name, to_f32(got), ref[i], ref[i + 3])


def test_cfg4_long_causal_full_size(oracle):
    from flame_amd import capi
    w = W.config4()
    B, H, S, _, D = w.shape
    assert (B, H, S, D) == (1, 32, 16384, 128) and w.causal
    print(f"[full] {w.name} shape={w.shape}", flush=True)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    q, k, v, do = (to_dev(t) for t in (w.q, w.k, w.v, w.do))
    o = torch.empty_like(q)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws_bytes = capi.bwd_workspace_bytes(B, H, S, D)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    _, lse = capi.attn_fwd(q, k, v, w.scale, causal=True, out=o)
    capi.attn_bwd(q, k, v, o, do, lse, w.scale, causal=True, workspace=ws, grads=(dq, dk, dv))
    torch.cuda.synchronize()
    tensors = 8 * q.numel() * 2 + lse.numel() * 4      # Q, K, V, dO, O, dQ, dK, dV
    peak = torch.cuda.max_memory_allocated() - base
    extra = peak - tensors
    print(f"      device memory: peak {peak / 2**20:.1f} MiB = 8 tensors + LSE {tensors / 2**20:.1f} MiB + {extra / 2**20:.1f} MiB "
          f"(declared workspace {ws_bytes / 2**20:.1f} MiB; a materialised bf16 P would be {H * S * S * 2 / 2**30:.0f} GiB)", flush=True)
    assert extra <= ws_bytes + (1 << 20)            # allocator rounding only; never O(S^2)
    assert ws_bytes <= 64 << 20

    # (a) oracle parity on row bands of the first and the last head
    go, glse = to_f32(o), lse.cpu().numpy().reshape(B, H, S)
    gdq, gdk, gdv = to_f32(dq), to_f32(dk), to_f32(dv)
    for hd in (0, H - 1):
        for r0 in (0, S // 2 - 64, S - 128):
            r1 = r0 + 128
            ro, rlse, ro32 = oracle.sdpa_fwd(w.q, w.k, w.v, w.scale, causal=True, heads=(hd, hd + 1), rows=(r0, r1),
                                             want_f32=True)
            assert_close_bf16(oracle, f"O head {hd} rows {r0}:{r1}", go[0, hd, r0:r1], ro[0, hd, r0:r1], ro32[0, hd, r0:r1])
            ml = oracle.max_abs(glse[0, hd, r0:r1], rlse[0, hd, r0:r1])
            print(f"      LSE head {hd} rows {r0}:{r1} max_abs={ml:.3e}", flush=True)
            assert ml <= TOL_LSE
            ref = oracle.sdpa_bwd(w.q, w.k, w.v, ro, w.do, w.scale, causal=True, heads=(hd, hd + 1), rows=(r0, r1),
                                  want_f32=True)
            assert_close_bf16(oracle, f"dQ head {hd} rows {r0}:{r1}", gdq[0, hd, r0:r1], ref[0][0, hd, r0:r1], ref[3][0, hd, r0:r1])
            if r1 == S:       # keys >= r0 are attended by the queries of this band only
                assert_close_bf16(oracle, f"dK head {hd} keys {r0}:{r1}", gdk[0, hd, r0:], ref[1][0, hd, r0:], ref[4][0, hd, r0:])
                assert_close_bf16(oracle, f"dV head {hd} keys {r0}:{r1}", gdv[0, hd, r0:], ref[2][0, hd, r0:], ref[5][0, hd, r0:])

    # (b) identities over all heads
    sum_dv = dv.double().sum(dim=2)
    sum_do = do.double().sum(dim=2)
    rel = float((sum_dv - sum_do).norm() / sum_do.norm())
    worst = float(((sum_dv - sum_do).norm(dim=-1) / sum_do.norm(dim=-1)).max())
    print(f"      sum_j dV_j vs sum_i dO_i: rel-L2 {rel:.3e}, worst head {worst:.3e}", flush=True)
    assert worst <= 1e-3
    sum_dk = dk.double().sum(dim=2).abs()
    abs_dk = dk.double().abs().sum(dim=2)
    ratio = float((sum_dk / abs_dk).max())
    print(f"      |sum_j dK_j| / sum_j |dK_j|: worst (head, channel) {ratio:.3e}", flush=True)
    assert ratio <= 1e-3
    assert bool(torch.isfinite(dq.float()).all()) and bool(torch.isfinite(dk.float()).all())
    # the last key of every head is attended by the last query alone: dV there is P * dO of that one pair,
    # with P = exp(s - LSE)
    last = S - 1
    s_last = (q[0, :, last].float() * k[0, :, last].float()).sum(-1) * w.scale
    p_last = torch.exp(s_last - lse.view(B, H, S)[0, :, last])
    want = p_last[:, None] * do[0, :, last].float()
    assert float((dv[0, :, last].float() - want).abs().max()) <= 2e-2
