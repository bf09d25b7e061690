"""Pins the CPU oracle of the element-wise tile primitives (oracle/tile_ops_oracle.c) without the GPU:
literal answers written out by hand, an independent numpy statement of each predicate, fp64 closed forms,
and the random generator against the xorshift recurrence evaluated in Python integers."""
import math

import numpy as np
import pytest

from oracle import oracle as O


def test_causal_mask_literal_and_offsets():
    s = np.arange(2 * 1 * 3 * 4, dtype=np.float32).reshape(2, 1, 3, 4)
    want = s.copy()
    M = np.float32(-1.0e9)
    # q_offset 1, k_offset 0: query row q sees keys 0 .. q+1
    want[:, :, 0, 2:] = M
    want[:, :, 1, 3:] = M
    got = O.tile_causal_mask(s.copy(), 1, 0)
    assert np.array_equal(got, want)
    # a tile to the right of the diagonal is masked whole, one far below it is untouched
    assert np.all(O.tile_causal_mask(s.copy(), 0, 100) == M)
    assert np.array_equal(O.tile_causal_mask(s.copy(), 100, 0), s)
    rng = np.random.default_rng(3)
    x = rng.normal(size=(2, 3, 17, 29)).astype(np.float32)
    qo, ko = 5, 9
    q = np.arange(17)[:, None] + qo
    k = np.arange(29)[None, :] + ko
    assert np.array_equal(O.tile_causal_mask(x.copy(), qo, ko), np.where(k > q, M, x))


def test_attn_mask_zero_excludes():
    rng = np.random.default_rng(4)
    x = rng.normal(size=(2, 2, 5, 7)).astype(np.float32)
    m = rng.integers(0, 3, size=x.shape).astype(np.uint8)       # 0, 1, 2: any non-zero byte keeps
    assert np.array_equal(O.tile_attn_mask(x.copy(), m), np.where(m == 0, np.float32(-1.0e9), x))


def test_add_mask_ranks_polarity_and_summation_order():
    rng = np.random.default_rng(5)
    BH, q_t, k_t, k_total, k0, q0 = 3, 4, 6, 20, 7, 9
    x = rng.normal(size=(BH, q_t, k_t)).astype(np.float32)
    N = np.float32(-1.0e30)
    # rank 3 boolean, zero excludes; rank 2 additive rows indexed by the absolute key
    b3 = rng.integers(0, 2, size=x.shape).astype(np.uint8)
    a2 = rng.normal(size=(BH, k_total)).astype(np.float32)
    want = x + ((np.float32(0) + a2[:, None, k0:k0 + k_t]) + np.where(b3 == 0, N, np.float32(0)))
    got = O.tile_add_mask(x.copy(), b3, a2, q0, k0, bool_rank=3, add_rank=2, k_total=k_total, zero_is_mask=True)
    assert np.array_equal(got, want.astype(np.float32))
    # rank 2 boolean with the other polarity, plus the causal term on absolute positions
    b2 = rng.integers(0, 2, size=(BH, k_total)).astype(np.uint8)
    kabs = k0 + np.arange(k_t)[None, None, :]
    qabs = q0 + np.arange(q_t)[None, :, None]
    delta = np.where(b2[:, None, k0:k0 + k_t] != 0, N, np.float32(0)).astype(np.float32)
    delta = (delta + np.where(kabs > qabs, N, np.float32(0))).astype(np.float32)
    got = O.tile_add_mask(x.copy(), b2, None, q0, k0, bool_rank=2, k_total=k_total, zero_is_mask=False, causal=True)
    assert np.array_equal(got, (x + delta).astype(np.float32))
    # both exclusions on one element add up to -2e30, not -1e30
    assert (got == np.float32(-2.0e30)).any() or not ((b2[:, None, k0:k0 + k_t] != 0) & (kabs > qabs)).any()
    # unknown ranks ignore the operand
    assert np.array_equal(O.tile_add_mask(x.copy(), b3, a2, bool_rank=1, add_rank=4, k_total=k_total), x)
    # order: delta = (0 + 1e30) + (-1e30) = 0 and the logit is unchanged; summed the other way round the logit
    # itself would be absorbed by 1e30 first
    one = np.full((1, 1, 1), 3.0, np.float32)
    add = np.full((1, 1, 1), 1.0e30, np.float32)
    excl = np.zeros((1, 1, 1), np.uint8)
    assert O.tile_add_mask(one.copy(), excl, add, bool_rank=3, add_rank=3)[0, 0, 0] == np.float32(3.0)


def test_lse_and_softmax_closed_forms():
    rng = np.random.default_rng(6)
    x = (rng.normal(size=(3, 5, 37)) * 4).astype(np.float32)
    lse = O.tile_lse_from_logits(x)
    ref = np.log(np.exp(x.astype(np.float64) - x.max(-1, keepdims=True)).sum(-1)) + x.max(-1)
    assert np.abs(lse - ref).max() <= 2e-6 * np.abs(ref).max()
    # one element: the element itself; shifting a row shifts its lse
    assert np.array_equal(O.tile_lse_from_logits(x[:, :, :1].copy()), x[:, :, 0])
    assert np.abs(O.tile_lse_from_logits(x + np.float32(8)) - (lse + 8)).max() <= 4e-6
    # no element at all, or only -inf: -inf
    assert np.all(O.tile_lse_from_logits(np.empty((1, 2, 0), np.float32)) == -np.inf)
    assert np.all(O.tile_lse_from_logits(np.full((1, 2, 3), -np.inf, np.float32)) == -np.inf)
    # softmax from the lse sums to one and equals exp(x - lse) in fp64 to fp32 accuracy
    bits, p32 = O.tile_softmax_from_lse(x, lse)
    assert np.abs(p32.astype(np.float64).sum(-1) - 1).max() <= 1e-5
    assert np.abs(p32 - np.exp(x.astype(np.float64) - lse[..., None].astype(np.float64))).max() <= 1e-6
    assert np.array_equal(bits, O.f32_to_bf16(p32))
    # merging the lse of two halves gives the lse of the row
    a = O.tile_lse_from_logits(np.ascontiguousarray(x[:, :, :20]))
    b = O.tile_lse_from_logits(np.ascontiguousarray(x[:, :, 20:]))
    assert np.abs(O.tile_lse_merge(a.copy(), b) - lse).max() <= 4e-6
    inf = np.full((2, 2), -np.inf, np.float32)
    assert np.all(O.tile_lse_merge(inf.copy(), inf) == -np.inf)
    assert np.array_equal(O.tile_lse_merge(inf.copy(), a[:2, :2].copy()), a[:2, :2])


def _uniform_by_hand(seed, b, qi, kj):
    m = 0xFFFFFFFF
    s = (seed & m) ^ ((1103515245 * (((b * 73856093) & m) ^ ((qi * 19349663) & m) ^ ((kj * 83492791) & m))) & m)
    s ^= (s << 13) & m
    s ^= s >> 17
    s ^= (s << 5) & m
    return (s & 0xFFFFFF) / 16777216.0


def test_dropout_generator_and_values():
    # the recurrence of sdpa_kernels.cu:18-33 in Python integers; 0x9E3779B97F4A7C15 also checks that only the
    # low 32 bits of the seed enter
    for seed, b, qi, kj in ((0, 0, 0, 0), (1, 0, 0, 0), (12345, 3, 17, 250), (0x9E3779B97F4A7C15, 47, 4607, 4607)):
        assert O.tile_uniform01(seed, b, qi, kj) == np.float32(_uniform_by_hand(seed, b, qi, kj))
    # seed 0 at the origin: the state is 0 and xorshift keeps it there
    assert O.tile_uniform01(0, 0, 0, 0) == 0.0
    rng = np.random.default_rng(7)
    BH, q_t, k_t, p, seed = 4, 33, 70, 0.3, 2024
    x = O.f32_to_bf16(rng.random(size=(BH, q_t, k_t)).astype(np.float32))
    got = O.tile_dropout(x.copy(), p, seed)
    u = np.array([[[_uniform_by_hand(seed, b, i, j) for j in range(k_t)] for i in range(q_t)] for b in range(BH)])
    drop = u.astype(np.float32) < np.float32(p)
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(p))
    want = O.f32_to_bf16(np.where(drop, np.float32(0), O.bf16_to_f32(x) * scale).astype(np.float32))
    assert np.array_equal(got, want)
    assert abs(drop.mean() - p) < 0.02
    # p = 0 keeps everything unchanged, p = 1 drops everything (scale 0)
    assert np.array_equal(O.tile_dropout(x.copy(), 0.0, seed), x)
    assert np.all(O.tile_dropout(x.copy(), 1.0, seed) == 0)
