"""Pins the CPU oracle (oracle/sdpa_oracle.c) before anything is compared against it.

None of these tests restates the oracle's own loops: each check is a reference known-answer
vector, an fp64 evaluation of the textbook definition, a library routine (torch CPU SDPA and
autograd), a finite difference, or an invariant that a plausible slip would break.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

from flame_amd import workloads as W

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _rand_bits(seed, shape, mul=1.0):
    return W.f32_to_bf16_bits(W.normal_f32(seed, 0, int(np.prod(shape))).reshape(shape) * np.float32(mul))


def test_bf16_round_to_nearest_even(oracle):
    # 1 + 2^-8 is a tie between 1.0 (even mantissa) and 1 + 2^-7: must go to even (1.0)
    x = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -1.0 - 2.0 ** -8], np.float32)
    bits = oracle.f32_to_bf16(x)
    back = oracle.bf16_to_f32(bits)
    assert back.tolist() == [1.0, 1.0 + 2.0 ** -6, 1.0 + 2.0 ** -7, -1.0]
    # agrees with torch's converter on random data, and with the product-side converter
    r = W.normal_f32(3, 1, 10000)
    t = torch.from_numpy(r).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(r), t)
    assert np.array_equal(W.f32_to_bf16_bits(r), t)


def test_reference_known_answer_2x2_masked(oracle):
    kat = json.load(open(os.path.join(GOLD, "kat_attention_2x2.json")))
    shp = (kat["B"], kat["H"], kat["Sq"], kat["D"])
    q = W.f32_to_bf16_bits(np.array(kat["q"], np.float32).reshape(shp))
    k = W.f32_to_bf16_bits(np.array(kat["k"], np.float32).reshape(shp))
    v = W.f32_to_bf16_bits(np.array(kat["v"], np.float32).reshape(shp))
    mask = np.array(kat["keep_mask"], np.uint8).reshape(1, 1, 2, 2)
    o, lse = oracle.sdpa_fwd(q, k, v, 1.0 / math.sqrt(kat["D"]), mask=mask)
    got = oracle.bf16_to_f32(o).ravel()
    assert np.max(np.abs(got - np.array(kat["expected_o"]))) < kat["tol"]
    # row 0 attends to key 0 only: its LSE is that single scaled logit
    s00 = (0.2 * 0.3 + -0.4 * 0.7) / math.sqrt(2.0)
    assert abs(lse[0, 0, 0] - s00) < 5e-3  # bf16 input rounding only


@pytest.mark.parametrize("case", [
    dict(B=2, H=3, Sq=17, Sk=29, D=8),
    dict(B=1, H=2, Sq=33, Sk=33, D=16, causal=True),
    dict(B=3, H=2, Sq=9, Sk=40, D=4, kv_len=[5, 40, 17]),
    dict(B=2, H=2, Sq=12, Sk=21, D=8, mask="full"),
    dict(B=2, H=2, Sq=12, Sk=21, D=8, mask="keypad", causal=True),
])
def test_forward_matches_fp64_definition(oracle, case):
    B, H, Sq, Sk, D = (case[x] for x in ("B", "H", "Sq", "Sk", "D"))
    q, k, v = (_rand_bits(11 + i, s) for i, s in enumerate([(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D)]))
    scale = 0.37
    keep = np.ones((B, H, Sq, Sk), bool)
    mask = None
    kv_len = case.get("kv_len")
    if case.get("causal"):
        keep &= np.arange(Sk)[None, :] <= np.arange(Sq)[:, None]
    if kv_len is not None:
        keep &= (np.arange(Sk)[None, :] < np.asarray(kv_len)[:, None])[:, None, None, :]
    if case.get("mask") == "full":
        mask = (W.normal_f32(5, 0, B * H * Sq * Sk).reshape(B, H, Sq, Sk) > -0.5).astype(np.uint8)
        mask[..., 0] = 1
        keep &= mask.astype(bool)
    if case.get("mask") == "keypad":
        mask = (W.normal_f32(6, 0, B * Sk).reshape(B, 1, 1, Sk) > -0.8).astype(np.uint8)
        mask[..., 0] = 1
        keep &= mask.astype(bool)
    o, lse, o32 = oracle.sdpa_fwd(q, k, v, scale, causal=case.get("causal", False), kv_len=kv_len,
                                  mask=mask, want_f32=True)
    O, LSE, P = oracle.brute_sdpa_f64(*(oracle.bf16_to_f32(t) for t in (q, k, v)), scale, keep)
    assert oracle.max_abs(o32, O) < 2e-5
    assert oracle.max_abs(lse, LSE) < 2e-5
    assert np.array_equal(o, oracle.f32_to_bf16(o32))
    # LSE identity: sum_j exp(s_ij - LSE_i) = 1 on every row with at least one attended key
    s = np.einsum("bhid,bhjd->bhij", *(oracle.bf16_to_f32(t).astype(np.float64) for t in (q, k))) * scale
    tot = np.where(keep, np.exp(s - lse[..., None].astype(np.float64)), 0.0).sum(-1)
    assert np.max(np.abs(tot - 1.0)) < 1e-5


def test_forward_matches_torch_cpu_sdpa(oracle):
    B, H, Sq, Sk, D = 2, 4, 64, 80, 32
    q, k, v = (_rand_bits(21 + i, s) for i, s in enumerate([(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D)]))
    tq, tk, tv = (torch.from_numpy(oracle.bf16_to_f32(t)) for t in (q, k, v))
    for causal in (False, True):
        ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=causal, scale=0.2)
        if causal:  # torch's causal mask is top-left aligned, like the reference's (k > q excluded)
            pass
        o, lse, o32 = oracle.sdpa_fwd(q, k, v, 0.2, causal=causal, want_f32=True)
        assert oracle.max_abs(o32, ref.numpy()) < 2e-5


def test_backward_matches_torch_cpu_autograd(oracle):
    B, H, Sq, Sk, D = 2, 2, 48, 56, 16
    shapes = [(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D), (B, H, Sq, D)]
    q, k, v, do = (_rand_bits(31 + i, s) for i, s in enumerate(shapes))
    kv_len = np.array([56, 23], np.int32)
    keep = (np.arange(Sk)[None, :] < kv_len[:, None])[:, None, None, :]
    tq, tk, tv = (torch.from_numpy(oracle.bf16_to_f32(t)).double().requires_grad_() for t in (q, k, v))
    ref = torch.nn.functional.scaled_dot_product_attention(
        tq, tk, tv, attn_mask=torch.from_numpy(np.broadcast_to(keep, (B, H, Sq, Sk)).copy()), scale=0.3)
    ref.backward(torch.from_numpy(oracle.bf16_to_f32(do)).double())
    o, lse = oracle.sdpa_fwd(q, k, v, 0.3, kv_len=kv_len)
    dq, dk, dv, dq32, dk32, dv32 = oracle.sdpa_bwd(q, k, v, o, do, 0.3, kv_len=kv_len, want_f32=True)
    # the oracle forms D from the bf16-rounded O: allow that rounding, nothing more
    for got, want in ((dq32, tq.grad), (dk32, tk.grad), (dv32, tv.grad)):
        assert oracle.rel_l2(got, want.numpy()) < 3e-3
        assert oracle.max_abs(got, want.numpy()) < 2e-2
    assert np.all(dk32[1, :, 23:, :] == 0) and np.all(dv32[1, :, 23:, :] == 0)
    assert np.array_equal(dq, oracle.f32_to_bf16(dq32))


def test_backward_matches_finite_differences(oracle):
    """Central differences of L = sum(O * dO) in fp64 on a 1x1x8x8x4 problem, causal."""
    Sq = Sk = 8
    D = 4
    shapes = [(1, 1, Sq, D), (1, 1, Sk, D), (1, 1, Sk, D), (1, 1, Sq, D)]
    q, k, v, do = (_rand_bits(41 + i, s) for i, s in enumerate(shapes))
    keep = (np.arange(Sk)[None, :] <= np.arange(Sq)[:, None])[None, None]
    f = [oracle.bf16_to_f32(t).astype(np.float64) for t in (q, k, v)]
    g = oracle.bf16_to_f32(do).astype(np.float64)
    scale = 0.5

    def loss(args):
        return float((oracle.brute_sdpa_f64(*args, scale, keep)[0] * g).sum())

    grads = []
    h = 1e-5
    for t in range(3):
        gr = np.zeros_like(f[t])
        it = np.nditer(f[t], flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            a = [x.copy() for x in f]
            b = [x.copy() for x in f]
            a[t][idx] += h
            b[t][idx] -= h
            gr[idx] = (loss(a) - loss(b)) / (2 * h)
        grads.append(gr)
    # un-rounded O for D here: feed the oracle an O that is exact in bf16? Not possible in general,
    # so compare with a tolerance that covers only the bf16 rounding of O (|dO||O| 2^-9 per term).
    o, _ = oracle.sdpa_fwd(q, k, v, scale, causal=True)
    _, _, _, dq32, dk32, dv32 = oracle.sdpa_bwd(q, k, v, o, do, scale, causal=True, want_f32=True)
    assert oracle.max_abs(dv32, grads[2]) < 1e-5          # dV does not involve D at all
    assert oracle.max_abs(dq32, grads[0]) < 1e-2 and oracle.rel_l2(dq32, grads[0]) < 1e-2
    assert oracle.max_abs(dk32, grads[1]) < 1e-2 and oracle.rel_l2(dk32, grads[1]) < 1e-2


def test_invariants(oracle):
    B, H, Sq, Sk, D = 1, 2, 16, 24, 8
    q, k, v = (_rand_bits(51 + i, s) for i, s in enumerate([(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D)]))
    o, lse, o32 = oracle.sdpa_fwd(q, k, v, 0.4, want_f32=True)
    perm = np.random.default_rng(0).permutation(Sk)
    o2, lse2, o32p = oracle.sdpa_fwd(q, k[:, :, perm], v[:, :, perm], 0.4, want_f32=True)
    assert oracle.max_abs(o32, o32p) < 1e-5 and oracle.max_abs(lse, lse2) < 1e-5
    vc = np.broadcast_to(v[:, :, :1, :], v.shape).copy()        # every value row identical
    o3, _ = oracle.sdpa_fwd(q, k, vc, 0.4)
    assert oracle.max_abs(oracle.bf16_to_f32(o3), np.broadcast_to(oracle.bf16_to_f32(vc[:, :, :1]), o3.shape)) < 1e-2
    # sum_j dS_ij = 0  <=>  dQ is unchanged when a constant is added to every dP row, i.e. when
    # V is shifted by a vector c along every key: dO.(V_j + c) = dP_ij + const_i
    do = _rand_bits(54, (B, H, Sq, D))
    dq_a = oracle.sdpa_bwd(q, k, v, o, do, 0.4, want_f32=True)[3]
    # shifting V changes O by c (bf16 rounding aside) and must leave dQ, dK unchanged
    shift = np.float32(0.25)
    v_s = oracle.f32_to_bf16(oracle.bf16_to_f32(v) + shift)
    o_s, _ = oracle.sdpa_fwd(q, k, v_s, 0.4)
    dq_b = oracle.sdpa_bwd(q, k, v_s, o_s, do, 0.4, want_f32=True)[3]
    assert oracle.rel_l2(dq_b, dq_a) < 2e-2


def test_fully_masked_rows(oracle):
    B, H, Sq, Sk, D = 1, 1, 4, 6, 4
    shapes = [(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D), (B, H, Sq, D)]
    q, k, v, do = (_rand_bits(61 + i, s) for i, s in enumerate(shapes))
    mask = np.ones((1, 1, Sq, Sk), np.uint8)
    mask[0, 0, 2, :] = 0
    o, lse = oracle.sdpa_fwd(q, k, v, 1.0, mask=mask)
    assert np.all(o[0, 0, 2] == 0) and lse[0, 0, 2] == -np.inf and np.all(np.isfinite(lse[0, 0, [0, 1, 3]]))
    dq, dk, dv = oracle.sdpa_bwd(q, k, v, o, do, 1.0, mask=mask)
    assert np.all(dq[0, 0, 2] == 0)
    assert np.all(np.isfinite(oracle.bf16_to_f32(dk))) and np.all(np.isfinite(oracle.bf16_to_f32(dv)))


def test_ragged_tail_is_excluded_not_zero_filled(oracle):
    """Reference regression tests/sdpa_ragged_sk.rs: Sk in {64,71,72,128,200}; a zero-filled tail
    would inflate the softmax denominator.  Checks kv_len against physically truncated K,V."""
    B, H, Sq, D = 1, 4, 64, 64
    for L in (64, 71, 72, 128, 200):
        Sk = 208
        q = _rand_bits(71, (B, H, Sq, D))
        k = _rand_bits(72, (B, H, Sk, D))
        v = _rand_bits(73, (B, H, Sk, D))
        a, la = oracle.sdpa_fwd(q, k, v, 0.125, kv_len=np.array([L], np.int32))
        b, lb = oracle.sdpa_fwd(q, k[:, :, :L].copy(), v[:, :, :L].copy(), 0.125)
        assert np.array_equal(a, b) and np.array_equal(la, lb)


def test_additive_bias_forward_against_torch_and_invariants(oracle):
    """softmax(scale*QK^T + bias) V: torch's CPU SDPA with a float attn_mask is the library check; a
    bias that is constant along each row must leave O unchanged; a bias of -1e9 where a keep-mask is 0
    must reproduce the keep-mask result (the reference's own masking arithmetic, src/sdpa.rs:458-470)."""
    import torch
    import torch.nn.functional as F
    B, H, Sq, Sk, D = 2, 3, 37, 53, 64
    q, k, v = (W.f32_to_bf16_bits(W.normal_f32(77, s, B * H * n * D).reshape(B, H, n, D))
               for s, n in enumerate((Sq, Sk, Sk)))
    bias = (W.normal_f32(77, 9, H * Sq * Sk).reshape(1, H, Sq, Sk) * np.float32(2.0)).astype(np.float32)
    scale = 0.3
    o, lse, o32 = oracle.sdpa_fwd_bias(q, k, v, scale, bias, want_f32=True)
    tq, tk, tv = (torch.from_numpy(W.bf16_bits_to_f32(t)) for t in (q, k, v))
    ref = F.scaled_dot_product_attention(tq, tk, tv, attn_mask=torch.from_numpy(bias), scale=scale).numpy()
    assert np.max(np.abs(o32 - ref)) < 2e-5
    s = np.einsum("bhqd,bhkd->bhqk", tq.numpy().astype(np.float64), tk.numpy().astype(np.float64)) * scale + bias
    assert np.max(np.abs(lse - np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) - s.max(-1))) < 1e-4
    # row-constant bias: softmax is shift invariant
    rowc = np.broadcast_to(W.normal_f32(78, 0, H * Sq).reshape(1, H, Sq, 1), (1, H, Sq, Sk)).copy()
    o_c, _ = oracle.sdpa_fwd_bias(q, k, v, scale, rowc)
    o_0, _ = oracle.sdpa_fwd(q, k, v, scale)
    assert np.max(np.abs(W.bf16_bits_to_f32(o_c) - W.bf16_bits_to_f32(o_0))) <= 2 ** -7
    # large negative bias == keep-mask
    keep = (np.random.default_rng(3).random((B, 1, Sq, Sk)) < 0.7).astype(np.uint8)
    keep[..., 0] = 1
    o_m, _ = oracle.sdpa_fwd(q, k, v, scale, mask=keep)
    o_b, _ = oracle.sdpa_fwd_bias(q, k, v, scale, ((1.0 - keep) * -1e9).astype(np.float32))
    assert np.array_equal(o_m, o_b)


def test_row_bands_equal_the_full_computation(oracle):
    """A band of query rows gives the rows of the full result bit for bit; under the causal flag the
    last band alone already holds the whole dK / dV of the keys that only it attends to."""
    B, H, S, D = 1, 3, 96, 8
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(41, s, B * H * S * D).reshape(B, H, S, D)) for s in range(4))
    scale = 0.3
    o, lse, o32 = oracle.sdpa_fwd(q, k, v, scale, causal=True, want_f32=True)
    dq, dk, dv, dq32, dk32, dv32 = oracle.sdpa_bwd(q, k, v, o, do, scale, causal=True, want_f32=True)
    for r0, r1 in ((0, 16), (40, 56), (80, 96)):
        bo, blse, bo32 = oracle.sdpa_fwd(q, k, v, scale, causal=True, heads=(1, 3), rows=(r0, r1), want_f32=True)
        assert np.array_equal(bo[0, 1:, r0:r1], o[0, 1:, r0:r1]) and np.array_equal(blse[0, 1:, r0:r1], lse[0, 1:, r0:r1])
        assert np.array_equal(bo32[0, 1:, r0:r1], o32[0, 1:, r0:r1])
        bo[0, 1:, r0:r1] = 0
        assert not bo.any()                      # nothing outside the band and the chosen heads is touched
        bdq, bdk, bdv, bdq32, _, bdv32 = oracle.sdpa_bwd(q, k, v, o, do, scale, causal=True, heads=(1, 3),
                                                         rows=(r0, r1), want_f32=True)
        assert np.array_equal(bdq[0, 1:, r0:r1], dq[0, 1:, r0:r1]) and np.array_equal(bdq32[0, 1:, r0:r1], dq32[0, 1:, r0:r1])
        if r1 == S:      # keys >= r0 are attended by queries >= r0 only
            assert np.array_equal(bdk[0, 1:, r0:], dk[0, 1:, r0:]) and np.array_equal(bdv[0, 1:, r0:], dv[0, 1:, r0:])
            assert not np.array_equal(bdv32[0, 1:, :r0], dv32[0, 1:, :r0])
    # the bands of a non-causal problem add up to the whole dK / dV
    _, _, _, _, dk32, dv32 = oracle.sdpa_bwd(q, k, v, o, do, scale, want_f32=True)
    parts = [oracle.sdpa_bwd(q, k, v, o, do, scale, rows=r, want_f32=True) for r in ((0, 50), (50, 96))]
    assert np.allclose(parts[0][4] + parts[1][4], dk32, atol=1e-5) and np.allclose(parts[0][5] + parts[1][5], dv32, atol=1e-5)
