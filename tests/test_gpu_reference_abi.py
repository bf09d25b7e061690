"""The entry points that keep the reference's own names and argument lists, called through ctypes the
way the reference's FFI declarations bind them, checked against the primary entry points / the oracle."""
import ctypes
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _i64x4(v):
    return (ctypes.c_int64 * 4)(*[int(x) for x in v])


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _z(n):
    return [ctypes.c_int64(0)] * n


def test_cudnn_named_trio_matches_reference_test_logic(oracle):
    """Shapes and seeds of tests/cudnn_sdpa_bwd_parity.rs:311-320: (1,4,128,64) and (1,4,256,128);
    train-forward O equals inference-forward O (ibid :250-308); grads against the fp32 recompute."""
    from flame_amd import capi
    lib = capi.lib()
    for (B, H, N, D) in ((1, 4, 128, 64), (1, 4, 256, 128)):
        t = [W.f32_to_bf16_bits(W.normal_f32(sd, 0, B * H * N * D).reshape(B, H, N, D)) for sd in (11, 22, 33, 44)]
        q, k, v, do = (to_dev(x) for x in t)
        scale = 1.0 / math.sqrt(D)
        st = _i64x4(q.stride())
        o_inf = torch.empty_like(q)
        o_trn = torch.empty_like(q)
        stats = torch.empty(B * H, N, dtype=torch.float32, device="cuda")
        assert lib.flame_cudnn_sdpa_bf16(_p(q), _p(k), _p(v), _p(o_inf), B, H, N, N, D, ctypes.c_float(scale),
                                         st, st, st, st, *_z(4), _stream()) == 0
        assert lib.flame_cudnn_sdpa_bf16_train_fwd(_p(q), _p(k), _p(v), _p(o_trn), _p(stats), B, H, N, N, D,
                                                   ctypes.c_float(scale), st, st, st, st, *_z(5), _stream()) == 0
        assert torch.equal(o_inf, o_trn)
        dq, dk, dv = (torch.empty_like(q) for _ in range(3))
        assert lib.flame_cudnn_sdpa_bwd_bf16(_p(q), _p(k), _p(v), _p(o_trn), _p(do), _p(stats), _p(dq), _p(dk), _p(dv),
                                             B, H, N, N, D, ctypes.c_float(scale), *([st] * 8), *_z(9), _stream()) == 0
        torch.cuda.synchronize()
        ro, rlse, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], scale, want_f32=True)
        ref = oracle.sdpa_bwd(t[0], t[1], t[2], ro, t[3], scale, want_f32=True)
        assert_close_bf16(oracle, "O", to_f32(o_trn), ro, ro32)
        assert oracle.max_abs(stats.cpu().numpy().reshape(rlse.shape), rlse) <= 1e-3
        for i, (name, g) in enumerate((("dQ", dq), ("dK", dk), ("dV", dv))):
            assert_close_bf16(oracle, name, to_f32(g), ref[i], ref[i + 3])
            # the reference's own gate (ibid :136-138): cosine >= 0.9999
            assert oracle.cosine(to_f32(g), ref[i + 3]) >= 0.9999


def test_flash_attention_symbol_fills_lse(oracle):
    """Shapes of tests/fa2_parity_naive.rs:374-376 (N in {512}, HD in {64,128}, 8 heads)."""
    from flame_amd import capi
    lib = capi.lib()
    for HD in (64, 128):
        BH, N = 8, 512
        t = [W.f32_to_bf16_bits(W.normal_f32(0xFA2 + HD, s, BH * N * HD).reshape(1, BH, N, HD)) for s in range(3)]
        q, k, v = (to_dev(x) for x in t)
        o = torch.empty_like(q)
        lse = torch.empty(BH, N, dtype=torch.float32, device="cuda")
        assert lib.flame_flash_attention_bf16(_p(q), _p(k), _p(v), _p(o), _p(lse), BH, N, N, HD, _stream()) == 0
        torch.cuda.synchronize()
        ro, rlse, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 1.0 / math.sqrt(HD), want_f32=True)
        ma, _ = assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
        assert ma <= 1e-2 and oracle.cosine(to_f32(o), ro32) >= 0.9999        # the reference's gate (:369-370)
        assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= 1e-3


def test_chunked_symbol_with_bf16_keep_mask_and_causal(oracle):
    from flame_amd import capi
    lib = capi.lib()
    lib.flame_sdpa_chunked_bf16.restype = ctypes.c_int
    B, H, Q, K, D = 2, 3, 40, 100, 64
    t = [W.f32_to_bf16_bits(W.normal_f32(321, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Q, K, K))]
    q, k, v = (to_dev(x) for x in t)
    keep = (W.normal_f32(322, 0, B * Q * K).reshape(B, 1, Q, K) > -0.2).astype(np.uint8)
    keep[..., 0] = 1
    mask_bf16 = torch.from_numpy(keep.astype(np.float32)).to(torch.bfloat16).cuda()
    out = torch.empty_like(q)
    # workspace sized the way the reference's caller sizes it: 4 * (chunk * K + chunk * (Dv + 2)) bytes
    # (cuda/src/flame_sdpa_stub.cu:973-976), far less than one byte per mask element times B*H
    chunk = 8
    ws = torch.empty(4 * (chunk * K + chunk * (D + 2)), dtype=torch.uint8, device="cuda")
    rc = lib.flame_sdpa_chunked_bf16(_p(q), _p(k), _p(v), B, H, Q, K, D, D, ctypes.c_float(0.125), chunk, 0, 1,
                                     _p(mask_bf16), _p(out), _p(ws), ctypes.c_uint64(ws.numel()), _stream())
    assert rc == 0
    torch.cuda.synchronize()
    ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, mask=keep, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(out), ro, ro32)
    # ... and with no workspace at all; a mask per head; mask together with the causal flag
    keep_h = (W.normal_f32(323, 0, B * H * Q * K).reshape(B, H, Q, K) > 0.1).astype(np.uint8)
    keep_h[..., 0] = 1
    mask_h = torch.from_numpy(keep_h.astype(np.float32)).to(torch.bfloat16).cuda()
    for causal in (0, 1):
        rc = lib.flame_sdpa_chunked_bf16(_p(q), _p(k), _p(v), B, H, Q, K, D, D, ctypes.c_float(0.125), 64, causal, H,
                                         _p(mask_h), _p(out), None, ctypes.c_uint64(0), _stream())
        assert rc == 0
        torch.cuda.synchronize()
        ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, causal=bool(causal), mask=keep_h, want_f32=True)
        assert_close_bf16(oracle, f"O per-head mask causal={causal}", to_f32(out), ro, ro32)
    # causal, no mask
    rc = lib.flame_sdpa_chunked_bf16(_p(q), _p(k), _p(v), B, H, Q, K, D, D, ctypes.c_float(0.125), 64, 1, 1,
                                     None, _p(out), None, ctypes.c_uint64(0), _stream())
    assert rc == 0
    torch.cuda.synchronize()
    ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, causal=True, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(out), ro, ro32)
    # a value head dim that is not a multiple of 8 (260): the reference's entry point takes any head dims, here such a
    # shape goes through the materialised path; checked against the oracle in column ranges of D (the softmax does not
    # depend on V)
    Dv = 260
    v_wide = W.f32_to_bf16_bits(W.normal_f32(4242, 9, B * H * K * Dv).reshape(B, H, K, Dv))
    out_wide = torch.full((B, H, Q, Dv), float("nan"), dtype=torch.bfloat16, device="cuda")
    vw = to_dev(v_wide)
    assert lib.flame_sdpa_chunked_bf16(_p(q), _p(k), _p(vw), B, H, Q, K, D, Dv, ctypes.c_float(0.125), 64, 0, 1,
                                       None, _p(out_wide), None, ctypes.c_uint64(0), _stream()) == 0
    torch.cuda.synchronize()
    for c0 in range(0, Dv, D):
        w = min(D, Dv - c0)
        vc = np.zeros((B, H, K, D), np.uint16)
        vc[..., :w] = v_wide[..., c0:c0 + w]
        ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], vc, 0.125, want_f32=True)
        assert_close_bf16(oracle, f"O columns {c0}..{c0 + w} of Dv = 260", to_f32(out_wide[..., c0:c0 + w]), ro[..., :w], ro32[..., :w])
    # bad chunk -> invalid (1): status enum of cuda/include/flame_cuda_status.h
    assert lib.flame_sdpa_chunked_bf16(_p(q), _p(k), _p(v), B, H, Q, K, D, D, ctypes.c_float(0.125), 0, 0, 1,
                                       None, _p(out), None, ctypes.c_uint64(0), _stream()) == 1


@pytest.mark.parametrize("Dh,Dv", [(64, 32), (64, 128), (96, 64), (40, 104), (64, 160), (64, 80), (128, 264)])
def test_value_head_dim_differs_from_query_head_dim(oracle, Dh, Dv):
    """V and O may have a head dim of their own in the chunked and streaming entry points
    (cuda/src/flame_sdpa_stub.cu:973-982, cuda/streaming_attn_bf16.h:7-17).  The oracle takes one head dim, so it
    is given both sides zero-padded to the larger one: zero channels change neither the logits nor the other
    channels of O."""
    from flame_amd import capi
    lib = capi.lib()
    lib.flame_sdpa_chunked_bf16.restype = ctypes.c_int
    B, H, Q, K = 2, 3, 150, 210
    q, k = (W.f32_to_bf16_bits(W.normal_f32(650 + Dh, s, B * H * n * Dh).reshape(B, H, n, Dh)) for s, n in ((0, Q), (1, K)))
    v = W.f32_to_bf16_bits(W.normal_f32(650 + Dv, 2, B * H * K * Dv).reshape(B, H, K, Dv))
    Dm = max(Dh, Dv)

    def pad(x):
        out = np.zeros(x.shape[:3] + (Dm,), np.uint16)
        out[..., :x.shape[3]] = x
        return out

    scale = 1.0 / math.sqrt(Dh)
    qd, kd, vd = to_dev(q), to_dev(k), to_dev(v)
    out = torch.full((B, H, Q, Dv), float("nan"), dtype=torch.bfloat16, device="cuda")
    for causal in (0, 1):
        rc = lib.flame_sdpa_chunked_bf16(_p(qd), _p(kd), _p(vd), B, H, Q, K, Dh, Dv, ctypes.c_float(scale), 64, causal, 1,
                                         None, _p(out), None, ctypes.c_uint64(0), _stream())
        assert rc == 0
        torch.cuda.synchronize()
        ro, _, ro32 = oracle.sdpa_fwd(pad(q), pad(k), pad(v), scale, causal=bool(causal), want_f32=True)
        assert_close_bf16(oracle, f"O chunked Dh={Dh} Dv={Dv} causal={causal}", to_f32(out), ro[..., :Dv], ro32[..., :Dv])
    # the streaming entry point (self-attention: one sequence length), strided
    S = K
    q2 = W.f32_to_bf16_bits(W.normal_f32(651 + Dh, 0, B * H * S * Dh).reshape(B, H, S, Dh))
    q2d = to_dev(q2)
    o2 = torch.full((B, H, S, Dv), float("nan"), dtype=torch.bfloat16, device="cuda")
    sq = [ctypes.c_long(x) for x in q2d.stride()]
    sk = [ctypes.c_long(x) for x in kd.stride()]
    sv = [ctypes.c_long(x) for x in vd.stride()]
    so = [ctypes.c_long(x) for x in o2.stride()]
    rc = lib.streaming_attn_bf16_fp32_launch(_p(q2d), _p(kd), _p(vd), B, H, S, Dh, Dv, *sq, *sk, *sv, _p(o2), *so,
                                             ctypes.c_float(scale), 128, 1, None, _stream())
    assert rc == 0
    torch.cuda.synchronize()
    ro, _, ro32 = oracle.sdpa_fwd(pad(q2), pad(k), pad(v), scale, causal=True, want_f32=True)
    assert_close_bf16(oracle, f"O streaming Dh={Dh} Dv={Dv}", to_f32(o2), ro[..., :Dv], ro32[..., :Dv])


def test_streaming_symbol_causal_and_key_padding(oracle):
    """Mirrors tests/streaming_attn.rs: small-sequence, causal, explicit key-padding mask."""
    from flame_amd import capi
    lib = capi.lib()
    B, H, S, D = 2, 2, 150, 64
    t = [W.f32_to_bf16_bits(W.normal_f32(555, s, B * H * S * D).reshape(B, H, S, D)) for s in range(3)]
    q, k, v = (to_dev(x) for x in t)
    o = torch.empty_like(q)
    st = [ctypes.c_long(x) for x in q.stride()]
    pad = (W.normal_f32(556, 0, B * H * S).reshape(B, H, S) > -0.5).astype(np.uint8)
    pad[..., 0] = 1
    padd = torch.from_numpy(pad).cuda()
    for causal, mask in ((0, None), (1, None), (0, padd), (1, padd)):
        rc = lib.streaming_attn_bf16_fp32_launch(_p(q), _p(k), _p(v), B, H, S, D, D, *st, *st, *st, _p(o), *st,
                                                 ctypes.c_float(0.125), 128, causal, _p(mask), _stream())
        assert rc == 0
        torch.cuda.synchronize()
        m4 = None if mask is None else pad.reshape(B, H, 1, S)
        ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, causal=bool(causal), mask=m4, want_f32=True)
        assert_close_bf16(oracle, f"O causal={causal} mask={mask is not None}", to_f32(o), ro, ro32)
    assert lib.streaming_attn_bf16_fp32_launch(_p(q), _p(k), _p(v), B, H, S, D, D, *st, *st, *st, _p(o), *st,
                                               ctypes.c_float(0.125), 0, 0, None, _stream()) != 0


def test_stream_symbol_takes_a_bf16_mask_where_one_means_excluded(oracle):
    """sdpa_stream_bf16_launch reads a bf16 mask through the caller's four element strides, and in this one
    entry point a value above 0.5 EXCLUDES (cuda/sdpa_stream_bf16.cu:79-81); the strides are those the
    reference's wrapper computes (src/cuda_ops_bf16.rs:1848-1873), 0 broadcasting heads or batches."""
    from flame_amd import capi
    lib = capi.lib()
    lib.sdpa_stream_bf16_launch.restype = ctypes.c_bool
    reason = ctypes.create_string_buffer(256)
    for D, (B, H, Q, K) in ((64, (2, 3, 96, 200)), (128, (1, 2, 130, 257))):
        t = [W.f32_to_bf16_bits(W.normal_f32(778 + D, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Q, K, K))]
        q, k, v = (to_dev(x) for x in t)
        o = torch.empty_like(q)
        for mh, mb in ((H, B), (1, B), (1, 1)):
            excl = (W.normal_f32(779, mh + 10 * mb, mb * mh * Q * K).reshape(mb, mh, Q, K) > 0.4).astype(np.uint8)
            excl[..., 0] = 0                       # the first key is never excluded
            excl[0, 0, 3, :] = 1                   # ... except for one row that loses every key
            m = torch.from_numpy(excl.astype(np.float32)).to(torch.bfloat16).cuda()
            strides = [1, K, 0 if mh == 1 else Q * K, 0 if mb == 1 else mh * Q * K]      # ek, eq, eh, eb
            ok = lib.sdpa_stream_bf16_launch(_p(q), _p(k), _p(v), _p(o), B, H, Q, K, D, ctypes.c_float(0.11), _p(m),
                                             *[ctypes.c_int64(x) for x in strides], 12, 96, 96, _stream(), reason, 256)
            assert ok and reason.value == b"", reason.value
            torch.cuda.synchronize()
            ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.11, mask=(1 - excl).astype(np.uint8), want_f32=True)
            assert_close_bf16(oracle, f"O D={D} mask heads={mh} batches={mb}", to_f32(o), ro, ro32)
            assert torch.all(o[0, 0, 3] == 0)


def test_stream_symbol_reports_reason_when_unsupported(oracle):
    from flame_amd import capi
    lib = capi.lib()
    lib.sdpa_stream_bf16_launch.restype = ctypes.c_bool
    B, H, Q, K, D = 1, 2, 96, 200, 64
    t = [W.f32_to_bf16_bits(W.normal_f32(777, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Q, K, K))]
    q, k, v = (to_dev(x) for x in t)
    o = torch.empty_like(q)
    reason = ctypes.create_string_buffer(256)
    ok = lib.sdpa_stream_bf16_launch(_p(q), _p(k), _p(v), _p(o), B, H, Q, K, D, ctypes.c_float(0.125), None,
                                     *_z(4), 12, 96, 96, _stream(), reason, 256)
    assert ok and reason.value == b""
    torch.cuda.synchronize()
    ro, _, ro32 = oracle.sdpa_fwd(t[0], t[1], t[2], 0.125, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o), ro, ro32)
    ok = lib.sdpa_stream_bf16_launch(_p(q), _p(k), _p(v), _p(o), B, H, Q, K, D, ctypes.c_float(0.125), None,
                                     *_z(4), 12, 128, 96, _stream(), reason, 256)
    assert not ok and b"q_tile" in reason.value


def test_cudnn_named_backward_on_two_streams_at_once():
    """flame_cudnn_sdpa_bwd_bf16 keeps its scratch per stream: calls of different shapes enqueued on two
    streams back to back, and a growing shape on a stream whose earlier call may still be running, give
    the results of the same calls made one at a time (same kernels and schedule: bit-identical)."""
    from flame_amd import capi

    def problem(seed, B, H, S, D):
        t = [to_dev(W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * S * D).reshape(B, H, S, D))) for s in range(4)]
        o, lse = capi.attn_fwd(t[0], t[1], t[2], 1.0 / math.sqrt(D))
        return (*t[:3], o, t[3], lse, 1.0 / math.sqrt(D))

    pa = problem(71, 1, 12, 3456, 128)     # splits its last dK/dV round: uses the partial-sum part of the scratch
    pb = problem(72, 2, 6, 1024, 64)
    pc = problem(73, 1, 16, 4096, 128)     # larger than pa: the scratch of pa's stream has to grow
    torch.cuda.synchronize()
    want = [capi.cudnn_sdpa_bwd(*p) for p in (pa, pb, pc)]
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got = [None, None, None]
    for _ in range(3):
        with torch.cuda.stream(s1):
            got[0] = capi.cudnn_sdpa_bwd(*pa)
        with torch.cuda.stream(s2):
            got[1] = capi.cudnn_sdpa_bwd(*pb)
        with torch.cuda.stream(s1):
            got[2] = capi.cudnn_sdpa_bwd(*pc)        # grows while pa may still be running on s1
        with torch.cuda.stream(s2):
            again = capi.cudnn_sdpa_bwd(*pb)
        torch.cuda.synchronize()
        for w_, g_ in zip(want, got):
            for a, b in zip(w_, g_):
                assert torch.equal(a, b)
        for a, b in zip(want[1], again):
            assert torch.equal(a, b)
