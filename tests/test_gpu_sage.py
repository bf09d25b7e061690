"""GPU parity of the SageAttention int8-QK path: quantised tensors and scales bit-exact against the
CPU oracle, output cosine >= 0.999 against the bf16 kernel on the same inputs."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import TOL_LSE, assert_close_bf16, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _check_quant(oracle, w, smooth=True):
    from flame_amd import capi
    q, k = to_dev(w.q), to_dev(w.k)
    got = capi.sage_quant(q, k, smooth_k=smooth)
    torch.cuda.synchronize()
    ref = oracle.sage_quant(w.q, w.k, smooth_k=smooth)
    assert np.array_equal(got["kmean"].cpu().numpy().view(np.uint32), ref["kmean"].view(np.uint32)), "kmean bits"
    assert np.array_equal(got["sq"].cpu().numpy().view(np.uint32), ref["sq"].view(np.uint32)), "sq bits"
    assert np.array_equal(got["sk"].cpu().numpy().view(np.uint32), ref["sk"].view(np.uint32)), "sk bits"
    assert np.array_equal(got["qi8"].cpu().numpy(), ref["qi8"]), "Q int8"
    assert np.array_equal(got["ki8"].cpu().numpy(), ref["ki8"]), "K int8"
    return got, ref


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("S", [64, 200, 384])
def test_quantisation_bit_exact_small(oracle, D, S):
    w = W.config5(B=1, H=3, S=S, D=D)
    print(f"[sage quant] S={S} D={D}", flush=True)
    _check_quant(oracle, w, smooth=True)
    _check_quant(oracle, w, smooth=False)


def test_quantisation_ties_and_zero_block(oracle):
    D = 64
    q = np.zeros((1, 1, 256, D), np.float32)
    q[0, 0, 0, :8] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]      # scale exactly 1: exact ties
    q[0, 0, 1, :4] = [-127.0, 126.5, -126.5, 0.25]
    k = np.zeros((1, 1, 128, D), np.float32)
    k[0, 0, :64, 0] = 1.0                                               # second K block is all zero
    w = W.Workload("ties", W.f32_to_bf16_bits(q), W.f32_to_bf16_bits(k), W.f32_to_bf16_bits(k), None, 1.0)
    got, ref = _check_quant(oracle, w, smooth=False)
    assert got["qi8"][0, 0, 0, :8].tolist() == [127, 0, 2, 2, 0, -2, -2, 4]
    assert float(got["sq"][0, 0, 1]) == 0.0 and torch.all(got["qi8"][0, 0, 128:] == 0)
    assert float(got["sk"][0, 0, 1]) == 0.0 and torch.all(got["ki8"][0, 0, 64:] == 0)


def test_quantisation_rounding_boundaries_and_tiny_scales(oracle):
    """The quantiser multiplies by 1/scale and falls back to the division only near a rounding boundary: blocks
    whose quotients sit on and next to k + 1/2 for scales that are not powers of two, and blocks so small that the
    scale is subnormal and its reciprocal overflows, must still give the codes of the IEEE quotient bit for bit."""
    D = 64
    rng = np.random.default_rng(17)
    q = np.zeros((1, 2, 512, D), np.float32)
    for blk, amax in enumerate((1.0, 3.0, 0.7109375, 254.0)):          # bf16-representable block maxima
        s = np.float32(amax) / np.float32(127.0)
        k = rng.integers(-126, 127, size=(128, D)).astype(np.float32)
        x = (k + np.float32(0.5)) * s                                   # on a boundary before the bf16 rounding ...
        x = W.bf16_bits_to_f32(W.f32_to_bf16_bits(x))                   # ... which moves it to either side, or not
        x[0, 0] = amax
        q[0, 0, 128 * blk:128 * (blk + 1)] = x
    tiny = np.float32(2.0 ** -120)
    q[0, 1, :128] = rng.integers(-64, 65, size=(128, D)).astype(np.float32) * tiny / 64
    q[0, 1, 128:256] = rng.integers(-3, 4, size=(128, D)).astype(np.float32) * np.float32(2.0 ** -126)
    kk = rng.normal(size=(1, 2, 128, D)).astype(np.float32) * np.float32(2.0 ** -118)
    w = W.Workload("boundaries", W.f32_to_bf16_bits(q), W.f32_to_bf16_bits(kk), W.f32_to_bf16_bits(kk), None, 1.0)
    _check_quant(oracle, w, smooth=True)
    _check_quant(oracle, w, smooth=False)


@pytest.mark.parametrize("D", [64, 128])
def test_sage_forward_small_against_oracle_and_bf16_path(oracle, D):
    from flame_amd import capi
    w = W.config5(B=1, H=2, S=328, D=D)
    print(f"[sage fwd] small D={D}", flush=True)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    qz = capi.sage_quant(q, k)
    o, lse = capi.sage_fwd(qz, v, w.scale, want_lse=True)
    o_bf16, lse_bf16 = capi.attn_fwd(q, k, v, w.scale)
    torch.cuda.synchronize()
    ref = oracle.sage_quant(w.q, w.k)
    ro, rlse, ro32 = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale, want_f32=True)
    # same quantised operands on both sides: only P->bf16 and accumulation order differ
    assert_close_bf16(oracle, "O_sage", to_f32(o), ro, ro32)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE
    cos = oracle.cosine(to_f32(o), to_f32(o_bf16))
    print(f"      cosine vs bf16 path = {cos:.6f}", flush=True)
    assert cos >= 0.999


def _check_sage_fwd(oracle, w, qz, ref, v, o_bf16, causal=False, kv_len=None):
    """int8-QK forward against the oracle run on the same quantised operands (north-star bar for a bf16
    output and for the log-sum-exp), and the cosine gate against the bf16 kernel beside it."""
    from flame_amd import capi
    kvl = None if kv_len is None else torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    o, lse = capi.sage_fwd(qz, v, w.scale, causal=causal, kv_len=kvl, want_lse=True)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale, causal=causal,
                                     kv_len=kv_len, want_f32=True)
    assert_close_bf16(oracle, f"O_sage causal={causal} kv_len={kv_len}", to_f32(o), ro, ro32)
    glse = lse.cpu().numpy().reshape(rlse.shape)
    fin = np.isfinite(rlse)
    assert np.array_equal(np.isfinite(glse), fin) and np.all(glse[~fin] == -np.inf)
    assert oracle.max_abs(glse[fin], rlse[fin]) <= TOL_LSE
    cos = oracle.cosine(to_f32(o), to_f32(o_bf16))
    print(f"      cosine vs bf16 path = {cos:.6f}", flush=True)
    assert cos >= 0.999


@pytest.mark.parametrize("D,S", [(64, 200), (128, 328)])
def test_sage_causal_and_key_length(oracle, D, S):
    from flame_amd import capi
    w = W.config5(B=2, H=2, S=S, D=D)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    qz = capi.sage_quant(q, k)
    ref = oracle.sage_quant(w.q, w.k)
    ref_c, _ = capi.attn_fwd(q, k, v, w.scale, causal=True)
    _check_sage_fwd(oracle, w, qz, ref, v, ref_c, causal=True)
    kv_len = [S, 77]
    kvl = torch.tensor(kv_len, dtype=torch.int32, device="cuda")
    ref_l, _ = capi.attn_fwd(q, k, v, w.scale, kv_len=kvl)
    _check_sage_fwd(oracle, w, qz, ref, v, ref_l, kv_len=kv_len)
    ref_cl, _ = capi.attn_fwd(q, k, v, w.scale, causal=True, kv_len=kvl)
    _check_sage_fwd(oracle, w, qz, ref, v, ref_cl, causal=True, kv_len=kv_len)


def test_sage_blocks_of_different_magnitude(oracle):
    """Q and K blocks scaled apart by up to 8x: a kernel that picked a block's scale by the wrong index
    would miss the oracle by far more than the tolerance."""
    from flame_amd import capi
    B, H, Sq, Sk, D = 1, 3, 328, 456, 128
    qf = W.normal_f32(61, 0, B * H * Sq * D).reshape(B, H, Sq, D)
    kf = W.normal_f32(61, 1, B * H * Sk * D).reshape(B, H, Sk, D)
    for ib, mul in enumerate((1.0, 3.0, 0.5)):
        qf[:, :, 128 * ib:128 * (ib + 1)] *= np.float32(mul)
    for jb, mul in enumerate((1.0, 2.0, 0.25, 1.5, 0.5, 2.0, 1.0, 0.125)):
        kf[:, :, 64 * jb:64 * (jb + 1)] *= np.float32(mul)
    w = W.Workload("sage_block_magnitudes", W.f32_to_bf16_bits(qf), W.f32_to_bf16_bits(kf),
                   W.f32_to_bf16_bits(W.normal_f32(61, 2, B * H * Sk * D).reshape(B, H, Sk, D)), None, 0.06)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    qz, ref = _check_quant(oracle, w, smooth=True)
    o_bf16, _ = capi.attn_fwd(q, k, v, w.scale)
    _check_sage_fwd(oracle, w, qz, ref, v, o_bf16)
    o_bf16c, _ = capi.attn_fwd(q, k, v, w.scale, causal=True)
    _check_sage_fwd(oracle, w, qz, ref, v, o_bf16c, causal=True)


@pytest.mark.parametrize("B,H,Sq,Sk,D", [(2, 16, 2048, 256, 64),      # 256 workgroups of 256 queries: whole rounds only
                                          (1, 36, 2048, 192, 64),      # 288: the last 32 are cut into 64 of 128 queries
                                          (1, 33, 2048, 320, 128),     # 264: the last 8 are cut into 16
                                          (2, 16, 2048, 64, 64),       # one key tile: prologue and a single step
                                          (2, 16, 1948, 128, 128),     # two key tiles; the last query tile is partly empty
                                          (1, 50, 1280, 576, 128)])    # 250 < compute units: 128-query workgroups only
def test_sage_large_problems_take_256_query_workgroups(oracle, B, H, Sq, Sk, D):
    """Problems without exclusions that fill the chip run 256-query workgroups, with a short last round cut into
    128-query workgroups: every head against the oracle, with Q blocks (128 rows) and K blocks (64 keys) scaled
    apart so that a scale taken from a neighbouring block, or a query tile mapped to the wrong rows, shows."""
    from flame_amd import capi
    qf = W.normal_f32(67, 0, B * H * Sq * D).reshape(B, H, Sq, D)
    kf = W.normal_f32(67, 1, B * H * Sk * D).reshape(B, H, Sk, D)
    for ib in range((Sq + 127) // 128):
        qf[:, :, 128 * ib:128 * (ib + 1)] *= np.float32((1.0, 3.0, 0.5, 2.0, 0.25)[ib % 5])
    for jb in range(Sk // 64):
        kf[:, :, 64 * jb:64 * (jb + 1)] *= np.float32((1.0, 2.0, 0.25, 1.5, 0.5, 2.0, 0.125)[jb % 7])
    w = W.Workload("sage_wide", W.f32_to_bf16_bits(qf), W.f32_to_bf16_bits(kf),
                   W.f32_to_bf16_bits(W.normal_f32(67, 2, B * H * Sk * D).reshape(B, H, Sk, D)), None, 0.5 / np.sqrt(D))
    print(f"[sage] {B}x{H} Sq={Sq} Sk={Sk} D={D}", flush=True)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    qz, ref = _check_quant(oracle, w, smooth=True)
    o_bf16, _ = capi.attn_fwd(q, k, v, w.scale)
    _check_sage_fwd(oracle, w, qz, ref, v, o_bf16)


def _rows_with_padding(t, D):
    """The [.., Dr] rows behind a [.., :D] view returned by capi.sage_quant."""
    from flame_amd import capi
    shape = tuple(t.shape[:-1]) + (capi.sage_row_elems(D),)
    return torch.as_strided(t, shape, t.stride(), t.storage_offset())


@pytest.mark.parametrize("D", [8, 40, 72, 96, 120])
def test_sage_other_head_dims(oracle, D):
    """Head dims that are not one of the two compiled sizes run on the next one with zero channels: codes, scales and
    channel means bit-exact on the D real channels, zero in the padding of every row the quantiser writes, the
    smoothed K bit-exact, and the int8 forward against the oracle on the same operands: plain, causal, with key
    lengths, and with an additive bias."""
    from flame_amd import capi
    B, H, Sq, Sk = 2, 2, 200, 328
    w = W.config5(B=B, H=H, S=Sk, D=D)
    qbits = w.q[:, :, :Sq].copy()
    wq = W.Workload("sage_d", qbits, w.k, w.v, None, w.scale)
    print(f"[sage] head dim {D}", flush=True)
    q, k, v = to_dev(qbits), to_dev(w.k), to_dev(w.v)
    for smooth in (True, False):
        got, ref = _check_quant(oracle, wq, smooth=smooth)
        for name in ("qi8", "ki8", "kmean"):
            assert torch.all(_rows_with_padding(got[name], D)[..., D:] == 0), f"{name} padding"
    qz = capi.sage_quant(q, k, want_ks=True)
    ref = oracle.sage_quant(qbits, w.k)
    assert np.array_equal(qz["ks"].cpu().contiguous().view(torch.int16).numpy().view(np.uint16), ref["ks"]), "smoothed K bits"
    assert torch.all(_rows_with_padding(qz["ks"], D)[..., D:].view(torch.int16) == 0)
    o_bf16, _ = capi.attn_fwd(q, k, v, w.scale)
    _check_sage_fwd(oracle, wq, qz, ref, v, o_bf16)
    o_c, _ = capi.attn_fwd(q, k, v, w.scale, causal=True)
    _check_sage_fwd(oracle, wq, qz, ref, v, o_c, causal=True)
    kv_len = [Sk, 77]
    o_l, _ = capi.attn_fwd(q, k, v, w.scale, kv_len=torch.tensor(kv_len, dtype=torch.int32, device="cuda"))
    _check_sage_fwd(oracle, wq, qz, ref, v, o_l, kv_len=kv_len)
    bias = (np.random.default_rng(5).normal(size=(1, H, Sq, Sk)) * 2).astype(np.float32)
    bias[..., 3::7] = -np.inf
    o, lse = capi.sage_fwd(qz, v, w.scale, bias=torch.from_numpy(bias).cuda(), want_lse=True)
    torch.cuda.synchronize()
    ro, rlse, ro32 = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale, bias=bias, want_f32=True)
    assert_close_bf16(oracle, f"O_sage bias D={D}", to_f32(o), ro, ro32)
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= TOL_LSE


def test_sage_head_dim_96_on_256_query_workgroups(oracle):
    """D = 96 on a problem that fills the chip (264 workgroups of 256 queries, the last 8 cut into 16): every head
    against the oracle."""
    from flame_amd import capi
    B, H, Sq, Sk, D = 1, 33, 2048, 320, 96
    w = W.Workload("sage_wide_d96", W.f32_to_bf16_bits(W.normal_f32(71, 0, B * H * Sq * D).reshape(B, H, Sq, D)),
                   W.f32_to_bf16_bits(W.normal_f32(71, 1, B * H * Sk * D).reshape(B, H, Sk, D)),
                   W.f32_to_bf16_bits(W.normal_f32(71, 2, B * H * Sk * D).reshape(B, H, Sk, D)), None, 1.0 / np.sqrt(D))
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    qz, ref = _check_quant(oracle, w, smooth=True)
    o_bf16, _ = capi.attn_fwd(q, k, v, w.scale)
    _check_sage_fwd(oracle, w, qz, ref, v, o_bf16)


def test_sage_refuses_head_dims_it_cannot_pad():
    from flame_amd import capi
    for D in (136, 20):
        q = torch.zeros((1, 1, 64, D), dtype=torch.bfloat16, device="cuda")
        with pytest.raises(capi.FlameAttnError):
            capi.sage_quant(q, q)


def test_sage_additive_bias_and_smoothed_k_output(oracle):
    """The attention_mask of the reference's Sage operator is added to the scores (src/sage_attention.rs:126-131):
    fp32 and bf16 biases, per head and broadcast, with excluded positions and a row that loses every key; and the
    smoothed K that the quantiser can hand back for a backward pass, bit-exact."""
    from flame_amd import capi
    B, H, Sq, Sk, D = 2, 3, 200, 328, 128
    w = W.config5(B=B, H=H, S=Sk, D=D)
    qbits = w.q[:, :, :Sq].copy()
    q, k, v = to_dev(qbits), to_dev(w.k), to_dev(w.v)
    qz = capi.sage_quant(q, k, want_ks=True)
    ref = oracle.sage_quant(qbits, w.k)
    assert np.array_equal(qz["ks"].cpu().view(torch.int16).numpy().view(np.uint16), ref["ks"]), "smoothed K bits"
    assert np.array_equal(qz["ki8"].cpu().numpy(), ref["ki8"])
    rng = np.random.default_rng(11)
    for shape, dt in (((B, H, Sq, Sk), torch.float32), ((1, H, Sq, Sk), torch.bfloat16), ((B, 1, Sq, Sk), torch.float32)):
        bias = (rng.normal(size=shape) * 2).astype(np.float32)
        bias[..., 5::9] = -np.inf
        bias[0, 0, 7, :] = -np.inf
        bt = torch.from_numpy(bias).cuda().to(dt)
        bias_seen = bt.float().cpu().numpy()             # what the kernel reads (bf16-rounded in the second case)
        for causal in (False, True):
            o, lse = capi.sage_fwd(qz, v, w.scale, causal=causal, bias=bt, want_lse=True)
            torch.cuda.synchronize()
            ro, rlse, ro32 = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale, causal=causal,
                                             bias=bias_seen, want_f32=True)
            assert_close_bf16(oracle, f"O_sage bias {shape} {dt} causal={causal}", to_f32(o), ro, ro32)
            glse = lse.cpu().numpy().reshape(rlse.shape)
            fin = np.isfinite(rlse)
            assert np.array_equal(np.isfinite(glse), fin) and np.all(glse[~fin] == -np.inf)
            assert oracle.max_abs(glse[fin], rlse[fin]) <= TOL_LSE
            assert torch.all(o[0, 0, 7] == 0)


def test_cfg5_production_shape(oracle):
    """B=2 H=24 S=4608 D=128: every int8 code and scale bit-exact; O cosine vs the bf16 kernel."""
    from flame_amd import capi
    w = W.config5()
    print("[sage] cfg5 full shape", flush=True)
    got, ref = _check_quant(oracle, w, smooth=True)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    o = capi.sage_fwd(got, v, w.scale)
    o_bf16, _ = capi.attn_fwd(q, k, v, w.scale)
    torch.cuda.synchronize()
    a, b = to_f32(o), to_f32(o_bf16)
    cos = oracle.cosine(a, b)
    per_head = min(oracle.cosine(a[i, j], b[i, j]) for i in range(a.shape[0]) for j in range(a.shape[1]))
    print(f"      cosine vs bf16 path: whole tensor {cos:.6f}, worst head {per_head:.6f}", flush=True)
    assert cos >= 0.999 and per_head >= 0.999
    # oracle parity of the int8 forward on two heads, O and log-sum-exp
    o2, lse2 = capi.sage_fwd(got, v, w.scale, want_lse=True)
    assert torch.equal(o2, o)
    for hd in (5, 47):
        ro, rlse, ro32 = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale, heads=(hd, hd + 1),
                                         want_f32=True)
        assert_close_bf16(oracle, f"O_sage head {hd}", a.reshape(48, 4608, 128)[hd], ro.reshape(48, 4608, 128)[hd],
                          ro32.reshape(48, 4608, 128)[hd])
        assert oracle.max_abs(lse2.cpu().numpy()[hd], rlse.reshape(48, 4608)[hd]) <= TOL_LSE
