"""Pins the oracle's dropout of the attention probabilities (the reference's autograd_v4 operator, unchunked:
src/autograd_v4/ops/sdpa.rs:229-231 and :600-649, generator src/rng/mod.rs:14-24) without the GPU: the kept set
against the xorshift recurrence in Python integers and in numpy, the forward against fp64 attention with that
set, the backward against fp64 central differences of the same function (the set is fixed by the seed, so the
function is smooth)."""
import numpy as np
import pytest

from oracle import oracle as O
from flame_amd import workloads as W


def _keep_by_hand(seed, idx, p):
    m = 0xFFFFFFFF
    s = (seed & m) ^ (idx & m)
    s ^= (s << 13) & m
    s ^= s >> 17
    s ^= (s << 5) & m
    return np.float32(s >> 8) * np.float32(1.0 / 16777216.0) >= np.float32(p)


def test_kept_set_follows_the_recurrence():
    for seed in (0, 1, 12345, 0x9E3779B97F4A7C15):
        for idx in (0, 1, 2, 1000, 2 ** 32 - 1, 2 ** 32 + 5, 24 * 4608 * 4608 - 1):
            for p in (0.1, 0.5):
                assert O.dropout_keep(seed, idx, p) == bool(_keep_by_hand(seed, idx, p)), (seed, idx, p)
    # index 2^32 + 5 and index 5 draw the same number: only the low 32 bits enter
    assert O.dropout_keep(7, 2 ** 32 + 5, 0.3) == O.dropout_keep(7, 5, 0.3)
    keep = O.dropout_keep_mask(2, 3, 17, 29, 0.25, 99)
    flat = keep.reshape(-1)
    for idx in (0, 5, 500, flat.size - 1):
        assert flat[idx] == bool(_keep_by_hand(99, idx, 0.25))
    # one xorshift round mixes poorly: over a few thousand neighbouring indices the kept fraction depends on the seed,
    # over a million it is 1 - p
    big = O.dropout_keep_mask(1, 4, 512, 512, 0.25, 4242)
    assert abs((~big).mean() - 0.25) < 0.01


@pytest.mark.parametrize("causal", [False, True])
def test_forward_with_dropout_against_fp64(causal):
    B, H, Sq, Sk, D, p, seed = 2, 3, 24, 40, 16, 0.3, 0x5DEECE66D
    q, k, v = (W.f32_to_bf16_bits(W.normal_f32(801, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Sq, Sk, Sk)))
    kv_len = np.array([Sk, 19], np.int32)
    keep_excl = np.broadcast_to((np.arange(Sk)[None, :] < kv_len[:, None])[:, None, None, :], (B, H, Sq, Sk)).copy()
    if causal:
        keep_excl &= (np.arange(Sk)[None, :] <= np.arange(Sq)[:, None])[None, None]
    f = [O.bf16_to_f32(t) for t in (q, k, v)]
    _, lse64, p64 = O.brute_sdpa_f64(*f, 0.25, keep_excl)
    m = O.dropout_keep_mask(B, H, Sq, Sk, p, seed)
    factor = np.float64(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))
    want = (p64 * m * factor) @ f[2].astype(np.float64)
    o, lse, o32 = O.sdpa_fwd_dropout(q, k, v, 0.25, p, seed, causal=causal, kv_len=kv_len, want_f32=True)
    assert np.abs(o32 - want).max() < 2e-5
    assert np.abs(lse - lse64).max() < 2e-5               # the log-sum-exp is that of the undropped softmax
    assert np.array_equal(o, O.f32_to_bf16(o32))
    # p = 0 is the plain forward, bit for bit
    o0, lse0 = O.sdpa_fwd_dropout(q, k, v, 0.25, 0.0, seed, causal=causal, kv_len=kv_len)
    o1, lse1 = O.sdpa_fwd(q, k, v, 0.25, causal=causal, kv_len=kv_len)
    assert np.array_equal(o0, o1) and np.array_equal(lse0, lse1)
    # a different seed drops a different set (seeds that differ in their low bits only permute the set within
    # small groups of neighbouring keys: the generator is one xorshift round of seed ^ index)
    o2, _ = O.sdpa_fwd_dropout(q, k, v, 0.25, p, seed ^ 0x9E3779B9, causal=causal, kv_len=kv_len)
    assert not np.array_equal(o2, o)
    assert 0.05 < m.mean() < 0.95       # small tensors: one xorshift round leaves the fraction far from 1 - p


def test_backward_with_dropout_against_finite_differences():
    Sq, Sk, D, seed, scale = 8, 10, 4, 0x2545F4914F6CDD1D, 0.5
    # one xorshift round gives neighbouring indices nearly the same uniform, so on a tensor this small a fixed p keeps
    # all or nothing: take p in the middle of the 160 uniforms, which splits them
    p = float(np.median(O.dropout_uniforms(1, 2, Sq, Sk, seed)))
    shapes = [(1, 2, Sq, D), (1, 2, Sk, D), (1, 2, Sk, D), (1, 2, Sq, D)]
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(811, i, int(np.prod(s))).reshape(s)) for i, s in enumerate(shapes))
    f = [O.bf16_to_f32(t).astype(np.float64) for t in (q, k, v)]
    g = O.bf16_to_f32(do).astype(np.float64)
    m = O.dropout_keep_mask(1, 2, Sq, Sk, p, seed)
    factor = np.float64(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))
    assert 0.05 < m.mean() < 0.95

    def loss(args):
        _, _, pr = O.brute_sdpa_f64(*args, scale)
        return float((((pr * m * factor) @ args[2]) * g).sum())

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
    o, _ = O.sdpa_fwd_dropout(q, k, v, scale, p, seed)
    _, _, _, dq32, dk32, dv32 = O.sdpa_bwd_dropout(q, k, v, o, do, scale, p, seed, want_f32=True)
    assert O.max_abs(dv32, grads[2]) < 1e-5               # dV does not involve the bf16-rounded O
    assert O.max_abs(dq32, grads[0]) < 1e-2 and O.rel_l2(dq32, grads[0]) < 1e-2
    assert O.max_abs(dk32, grads[1]) < 1e-2 and O.rel_l2(dk32, grads[1]) < 1e-2
    # teeth: the gradient of the undropped function is far from these
    _, _, _, dq_plain, _, dv_plain = O.sdpa_bwd(q, k, v, O.sdpa_fwd(q, k, v, scale)[0], do, scale, want_f32=True)
    assert O.rel_l2(dv_plain, grads[2]) > 0.1 and O.rel_l2(dq_plain, grads[0]) > 0.1


# ------------------------------------------------------------------------------------------ the chunked draw
def _tile_keep_by_hand(seed, bh, i, j, Sq, Sk, cq, ck, p):
    """derive_tile_seed and the tile's own flat index in Python integers (src/autograd_v4/ops/sdpa.rs:600-602, :604-649):
    the tile tensor is [B*H, q_t, k_t], its seed (seed + ((q_offset << 32) ^ k_offset)) truncated to 32 bits."""
    q_off, k_off = (i // cq) * cq, (j // ck) * ck
    q_t, k_t = min(cq, Sq - q_off), min(ck, Sk - k_off)
    tile_seed = ((seed + ((q_off << 32) ^ k_off)) & (2 ** 64 - 1)) & 0xFFFFFFFF
    return _keep_by_hand(tile_seed, (bh * q_t + (i - q_off)) * k_t + (j - k_off), p)


def test_chunked_draw_follows_the_tile_seeds_and_indices():
    seed, Sq, Sk, cq, ck = 0x2545F4914F6CDD1D, 10, 7, 4, 3
    # written out once: element (bh 2, query 9, key 6) lies in the tile at offsets (8, 6) of size 2 x 1, where it has
    # flat index (2 * 2 + 1) * 1 + 0 = 5, and the tile's seed is the low word of seed + 6 (the query offset is shifted
    # out of it)
    assert ((seed + ((8 << 32) ^ 6)) & 0xFFFFFFFF) == ((seed & 0xFFFFFFFF) + 6) & 0xFFFFFFFF
    for p in (0.2, 0.5, 0.8):
        assert O.dropout_keep_tiled(seed, 2, 9, 6, Sq, Sk, cq, ck, p) == bool(_keep_by_hand((seed & 0xFFFFFFFF) + 6, 5, p))
    u = O.dropout_uniforms(2, 2, Sq, Sk, seed, cq, ck).reshape(4, Sq, Sk)
    for p in (0.3, 0.6):
        for bh in range(4):
            for i in range(Sq):
                for j in range(Sk):
                    want = bool(_tile_keep_by_hand(seed, bh, i, j, Sq, Sk, cq, ck, p))
                    assert O.dropout_keep_tiled(seed, bh, i, j, Sq, Sk, cq, ck, p) == want
                    assert bool(u[bh, i, j] >= np.float32(p)) == want
    # chunks that cover the whole axes are the unchunked draw; a chunk along the queries alone changes the indices only
    assert np.array_equal(O.dropout_uniforms(2, 2, Sq, Sk, seed, Sq, Sk), O.dropout_uniforms(2, 2, Sq, Sk, seed))
    assert np.array_equal(O.dropout_uniforms(2, 2, Sq, Sk, seed, 100, 0), O.dropout_uniforms(2, 2, Sq, Sk, seed))
    assert not np.array_equal(O.dropout_uniforms(2, 2, Sq, Sk, seed, 4, 0), O.dropout_uniforms(2, 2, Sq, Sk, seed))
    # a low seed word that wraps with the key offset
    s2 = 0xFFFFFFFF_FFFFFFFE
    assert O.dropout_keep_tiled(s2, 0, 1, 5, 4, 8, 2, 4, 0.5) == bool(_keep_by_hand((0xFFFFFFFE + 4) & 0xFFFFFFFF, (0 * 2 + 1) * 4 + 1, 0.5))


def test_forward_and_backward_with_a_chunked_draw_against_fp64():
    B, H, Sq, Sk, D, seed, cq, ck = 1, 2, 12, 20, 8, 0x5DEECE66D, 5, 8
    p = float(np.median(O.dropout_uniforms(B, H, Sq, Sk, seed, cq, ck)))
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(821, s, B * H * n * D).reshape(B, H, n, D)) for s, n in enumerate((Sq, Sk, Sk, Sq)))
    f = [O.bf16_to_f32(t).astype(np.float64) for t in (q, k, v)]
    g = O.bf16_to_f32(do).astype(np.float64)
    m = O.dropout_keep_mask(B, H, Sq, Sk, p, seed, cq, ck)
    assert not np.array_equal(m, O.dropout_keep_mask(B, H, Sq, Sk, p, seed)) and 0.05 < m.mean() < 0.95
    factor = np.float64(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))
    _, lse64, p64 = O.brute_sdpa_f64(*f, 0.3)
    pd = p64 * m * factor
    o, lse, o32 = O.sdpa_fwd_dropout(q, k, v, 0.3, p, seed, want_f32=True, chunk_q=cq, chunk_kv=ck)
    assert np.abs(o32 - pd @ f[2]).max() < 2e-5 and np.abs(lse - lse64).max() < 2e-5
    # closed-form gradients of sum(g * (P m f) V) in fp64, with the oracle's D = rowsum(dO * O_bf16) convention
    _, _, _, dq32, dk32, dv32 = O.sdpa_bwd_dropout(q, k, v, o, do, 0.3, p, seed, want_f32=True, chunk_q=cq, chunk_kv=ck)
    dv = np.swapaxes(pd, -1, -2) @ g
    dpd = g @ np.swapaxes(f[2], -1, -2)
    dp = dpd * m * factor
    delta = (g * O.bf16_to_f32(o).astype(np.float64)).sum(-1, keepdims=True)
    ds = p64 * (dp - delta) * 0.3
    assert O.max_abs(dv32, dv) < 1e-5
    assert O.max_abs(dq32, ds @ f[1]) < 1e-5 and O.max_abs(dk32, np.swapaxes(ds, -1, -2) @ f[0]) < 1e-5


def test_operand_rounding_variant_rounds_exactly_the_matrix_operands():
    """oracle.operand_rounding(): P f before P V and P^T dO, and dS before dS K and dS^T Q, are rounded to bf16 and
    nothing else is.  Pinned by recomputing the four products in fp64 from operands rounded here with
    oracle.f32_to_bf16 (taken from the fp64 softmax, so the check does not reuse the oracle's own P), on a case where
    the rounding is visible; and by the switch restoring the plain values."""
    B, H, Sq, Sk, D, seed, scale = 1, 2, 12, 9, 8, 0x2545F4914F6CDD1D, 0.4
    p = float(np.quantile(O.dropout_uniforms(B, H, Sq, Sk, seed), 0.3))
    shapes = [(B, H, Sq, D), (B, H, Sk, D), (B, H, Sk, D), (B, H, Sq, D)]
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(821, i, int(np.prod(s))).reshape(s)) for i, s in enumerate(shapes))
    fq, fk, fv, g = (O.bf16_to_f32(t).astype(np.float64) for t in (q, k, v, do))
    _, _, pr = O.brute_sdpa_f64(fq, fk, fv, scale)
    m = O.dropout_keep_mask(B, H, Sq, Sk, p, seed)
    factor = np.float64(np.float32(1.0) / (np.float32(1.0) - np.float32(p)))

    def rb(x):        # round to bf16, back to fp64
        return O.bf16_to_f32(O.f32_to_bf16(x.astype(np.float32))).astype(np.float64)

    pt = rb(pr * m * factor)
    want_o = pt @ fv
    plain = O.sdpa_fwd_dropout(q, k, v, scale, p, seed, want_f32=True)
    with O.operand_rounding():
        ro, _, ro32 = O.sdpa_fwd_dropout(q, k, v, scale, p, seed, want_f32=True)
        _, _, _, dq32, dk32, dv32 = O.sdpa_bwd_dropout(q, k, v, ro, do, scale, p, seed, want_f32=True)
    again = O.sdpa_fwd_dropout(q, k, v, scale, p, seed, want_f32=True)
    assert np.array_equal(plain[2], again[2])                      # the switch is off again
    assert np.abs(ro32 - want_o).max() < 5e-6
    assert np.abs(plain[2] - want_o).max() > 1e-4                  # ... and the rounding is visible in this case
    delta = (g * O.bf16_to_f32(ro).astype(np.float64)).sum(-1, keepdims=True)
    ds = rb(pr * (m * factor * (g @ fv.transpose(0, 1, 3, 2)) - delta))
    assert np.abs(dv32 - pt.transpose(0, 1, 3, 2) @ g).max() < 5e-6
    # dS is rounded from fp32 values that differ from the fp64 ones in their last bits: a rounding that falls the
    # other way moves a product by one bf16 step of dS times an element of K or Q, so these two are held less tightly
    assert np.abs(dq32 - scale * (ds @ fk)).max() < 2e-2 and O.rel_l2(dq32, scale * (ds @ fk)) < 2e-3
    assert np.abs(dk32 - scale * (ds.transpose(0, 1, 3, 2) @ fq)).max() < 2e-2 and O.rel_l2(dk32, scale * (ds.transpose(0, 1, 3, 2) @ fq)) < 2e-3
