"""GPU parity of the tiled forward (O and log-sum-exp) against the CPU oracle, through the C ABI."""
import json
import math
import os

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_bits, to_dev, to_f32

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _check_fwd(oracle, w, heads=None, tag=""):
    from flame_amd import capi
    print(f"[fwd] {w.name} {tag} shape={w.shape} causal={w.causal}", flush=True)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    kvl = None if w.kv_len is None else torch.from_numpy(w.kv_len).cuda()
    mask = None if w.mask is None else torch.from_numpy(w.mask).cuda()
    o, lse = capi.attn_fwd(q, k, v, w.scale, causal=w.causal, kv_len=kvl, mask=mask)
    torch.cuda.synchronize()
    B, H, Sq, Sk, D = w.shape
    ro, rlse, ro32 = oracle.sdpa_fwd(w.q, w.k, w.v, w.scale, causal=w.causal, kv_len=w.kv_len, mask=w.mask,
                                     heads=heads, want_f32=True)
    go = to_f32(o).reshape(B * H, Sq, D)
    glse = lse.cpu().numpy()
    rlse = rlse.reshape(B * H, Sq)
    hb, he = (0, B * H) if heads is None else heads
    go, glse, rlse = go[hb:he], glse[hb:he], rlse[hb:he]
    assert_close_bf16(oracle, "O", go, ro.reshape(B * H, Sq, D)[hb:he], ro32.reshape(B * H, Sq, D)[hb:he])
    fin = np.isfinite(rlse)
    assert np.array_equal(np.isfinite(glse), fin)
    assert np.all(glse[~fin] == -np.inf)
    ml = oracle.max_abs(glse[fin], rlse[fin])
    print(f"      LSE max_abs={ml:.3e}", flush=True)
    assert ml <= TOL_LSE
    return o, lse


def test_cfg1_small_noncausal(oracle):
    _check_fwd(oracle, W.config1())


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (2, 2), (37, 91), (128, 64), (129, 193), (300, 257)])
def test_partial_tiles(oracle, D, Sq, Sk):
    seed = 1000 + Sq * 7 + Sk
    B, H = 2, 3
    t = [W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D))
         for s, n in enumerate((Sq, Sk, Sk))]
    w = W.Workload(f"partial_{Sq}x{Sk}_d{D}", t[0], t[1], t[2], None, 1.0 / math.sqrt(D))
    _check_fwd(oracle, w)


@pytest.mark.parametrize("D", [64, 128])
def test_causal(oracle, D):
    _check_fwd(oracle, W.config4(H=2, S=320, D=D))


def test_causal_rectangular(oracle):
    # more keys than queries and the reverse: key j > query i is excluded (top-left aligned)
    for Sq, Sk in ((100, 260), (260, 100)):
        t = [W.f32_to_bf16_bits(W.normal_f32(5 + Sq, s, 2 * n * 64).reshape(1, 2, n, 64))
             for s, n in enumerate((Sq, Sk, Sk))]
        _check_fwd(oracle, W.Workload(f"causal_rect_{Sq}x{Sk}", t[0], t[1], t[2], None, 0.125, causal=True))


def test_cfg3_ragged_key_lengths(oracle):
    w = W.config3(H=2, Sq=192)
    o, lse = _check_fwd(oracle, w)
    # the same exclusions expressed as a [B,1,1,Sk] keep-mask: same result up to rounding (the masked
    # body walks every key tile, the key-length body stops at the last attended one), same parity bar
    w2 = W.Workload("cfg3_as_keep_mask", w.q, w.k, w.v, None, w.scale, mask=w.extra["keep_mask"])
    o2, lse2 = _check_fwd(oracle, w2)
    assert oracle.max_abs(to_f32(o), to_f32(o2)) <= 1e-2


def test_reference_ragged_regression_shapes(oracle):
    """Sk in {64,71,72,128,200}, B=1 H=32 Sq=64 D=64 (reference tests/sdpa_ragged_sk.rs:126-163)."""
    for Sk in (64, 71, 72, 128, 200):
        t = [W.f32_to_bf16_bits(W.normal_f32(900 + Sk, s, 32 * n * 64).reshape(1, 32, n, 64))
             for s, n in enumerate((64, Sk, Sk))]
        _check_fwd(oracle, W.Workload(f"ragged_sk{Sk}", t[0], t[1], t[2], None, 0.125))


def test_general_keep_mask_and_fully_masked_rows(oracle):
    B, H, Sq, Sk, D = 2, 2, 70, 150, 64
    t = [W.f32_to_bf16_bits(W.normal_f32(77, s, B * H * n * D).reshape(B, H, n, D))
         for s, n in enumerate((Sq, Sk, Sk))]
    mask = (W.normal_f32(78, 0, B * H * Sq * Sk).reshape(B, H, Sq, Sk) > 0.3).astype(np.uint8)
    mask[0, 1, 5, :] = 0            # a fully excluded row: O = 0, LSE = -inf
    mask[1, 0, 69, :] = 0
    w = W.Workload("general_mask", t[0], t[1], t[2], None, 0.2, mask=mask)
    o, lse = _check_fwd(oracle, w)
    assert torch.all(o[0, 1, 5] == 0) and torch.all(o[1, 0, 69] == 0)
    # broadcast over heads and batch: [1,1,Sq,Sk]
    w2 = W.Workload("bcast_mask", t[0], t[1], t[2], None, 0.2, mask=mask[:1, :1].copy())
    _check_fwd(oracle, w2)


def test_reference_known_answer_2x2(oracle):
    """Reference KAT (src/tests/attention_tests.rs:110-155), head dim 2 zero-padded to 64."""
    from flame_amd import capi
    kat = json.load(open(os.path.join(GOLD, "kat_attention_2x2.json")))

    def pad(vals):
        a = np.zeros((1, 1, 2, 64), np.float32)
        a[0, 0, :, :2] = np.array(vals, np.float32).reshape(2, 2)
        return to_dev(W.f32_to_bf16_bits(a))

    mask = torch.tensor(kat["keep_mask"], dtype=torch.uint8).reshape(1, 1, 2, 2).cuda()
    o, _ = capi.attn_fwd(pad(kat["q"]), pad(kat["k"]), pad(kat["v"]), 1.0 / math.sqrt(2.0), mask=mask)
    got = to_f32(o)[0, 0, :, :2].ravel()
    assert np.max(np.abs(got - np.array(kat["expected_o"]))) < kat["tol"]
    assert torch.all(o[0, 0, :, 2:] == 0)


def test_strided_views_match_contiguous(oracle):
    """The DiT layout reshape([B,N,H,D]).permute(0,2,1,3) runs without a copy (reference src/sdpa.rs:607-621)."""
    from flame_amd import capi
    w = W.config2(H=3, n_text=40, grid=12, D=128)       # 184 tokens
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    o_ref, lse_ref = capi.attn_fwd(q, k, v, w.scale)
    qs, ks, vs = (t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3) for t in (q, k, v))
    assert not qs.is_contiguous()
    out = torch.empty_like(qs.permute(0, 2, 1, 3).contiguous()).permute(0, 2, 1, 3)
    o2, lse2 = capi.attn_fwd(qs, ks, vs, w.scale, out=out)
    assert torch.equal(o2, o_ref) and torch.equal(lse2, lse_ref)
    _check_fwd(oracle, w)


def test_cfg2_production_shape_head_subset(oracle):
    """Full B=1 H=24 S=4608 D=128 launch; oracle parity on two heads keeps the CPU time bounded."""
    w = W.config2()
    _check_fwd(oracle, w, heads=(0, 1), tag="head 0")
    _check_fwd(oracle, w, heads=(23, 24), tag="head 23")


@pytest.mark.parametrize("D,H,Sq,Sk", [(128, 64, 1024, 512), (64, 64, 1024, 256), (128, 3, 200, 512)])
def test_reference_maximum_moves_during_the_walk(oracle, D, H, Sq, Sk):
    """Later keys carry far larger logits than the first tile, so the running maximum outgrows the stale
    reference by more than 2^8 several times and O is rescaled mid-walk; the first two shapes fill 256-query
    workgroups on every compute unit (the one-wavefront-per-SIMD kernels), the third uses the narrow ones."""
    seed = 4242 + D + Sq
    B = 1
    t = [W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D) for s, n in enumerate((Sq, Sk, Sk))]
    k = t[1]
    for j, f in ((64, 4.0), (192, 12.0), (Sk - 64, 30.0)):     # logits grow in steps along the key axis
        k[:, :, j:, :] *= f / (k[:, :, j:j + 1, :].std() + 1e-6) * k[:, :, :64, :].std()
    bits = [W.f32_to_bf16_bits(x) for x in (t[0], k, t[2])]
    w = W.Workload(f"maxmove_{Sq}x{Sk}_d{D}_h{H}", bits[0], bits[1], bits[2], None, 1.0 / math.sqrt(D))
    _check_fwd(oracle, w, heads=(0, min(H, 3)))


def test_invalid_arguments_are_rejected():
    from flame_amd import capi
    for bad_d in (100, 132, 520):                          # not a multiple of 8, or above 512
        q = torch.zeros(1, 1, 8, bad_d, dtype=torch.bfloat16, device="cuda")
        with pytest.raises(capi.FlameAttnError) as e:
            capi.attn_fwd(q, q, q, 0.1)
        assert e.value.code == capi.ERR_UNSUPPORTED
    q = torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(capi.FlameAttnError) as e:
        capi.attn_fwd(q, q, q, -1.0)
    assert e.value.code == capi.ERR_INVALID
    with pytest.raises(capi.FlameAttnError) as e:
        capi.attn_fwd(q.transpose(2, 3), q, q, 0.1)         # D stride != 1
    assert e.value.code in (capi.ERR_UNSUPPORTED, capi.ERR_INVALID)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("bias_dtype", ["f32", "bf16"])
def test_additive_bias(oracle, D, bias_dtype):
    """softmax(scale*QK^T + bias) V with a [1,H,Sq,Sk] relative-position style bias."""
    from flame_amd import capi
    B, H, Sq, Sk = 2, 3, 200, 333
    print(f"[fwd bias] D={D} bias={bias_dtype}", flush=True)
    q, k, v = (W.f32_to_bf16_bits(W.normal_f32(91, s, B * H * n * D).reshape(B, H, n, D))
               for s, n in enumerate((Sq, Sk, Sk)))
    bias = (W.normal_f32(91, 7, H * Sq * Sk).reshape(1, H, Sq, Sk) * np.float32(1.5)).astype(np.float32)
    if bias_dtype == "bf16":
        bias_bits = W.f32_to_bf16_bits(bias)
        bias = W.bf16_bits_to_f32(bias_bits)
        bd = to_dev(bias_bits)
    else:
        bd = torch.from_numpy(bias).cuda()
    scale = 1.0 / math.sqrt(D)
    o, lse = capi.attn_fwd_bias(to_dev(q), to_dev(k), to_dev(v), scale, bd)
    torch.cuda.synchronize()
    ro, rlse, rof = oracle.sdpa_fwd_bias(q, k, v, scale, bias, want_f32=True)
    assert_close_bf16(oracle, "O", to_f32(o), ro, rof)
    assert np.max(np.abs(lse.cpu().numpy().reshape(rlse.shape) - rlse)) <= TOL_LSE
    # with a keep-mask on top
    keep = (np.random.default_rng(5).random((B, 1, Sq, Sk)) < 0.5).astype(np.uint8)
    keep[..., 0] = 1
    o2, _ = capi.attn_fwd_bias(to_dev(q), to_dev(k), to_dev(v), scale, bd, mask=torch.from_numpy(keep).cuda())
    torch.cuda.synchronize()
    ro2, _, rof2 = oracle.sdpa_fwd_bias(q, k, v, scale, (bias + (1.0 - keep) * np.float32(-1e9)).astype(np.float32),
                                        want_f32=True)
    assert_close_bf16(oracle, "O masked", to_f32(o2), ro2, rof2)
