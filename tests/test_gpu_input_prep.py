"""GPU parity of the fused input preparation (RMS-norm + RoPE + layout change) against the oracle: bit-identical.

Every step of the kernel is IEEE arithmetic with the oracle's roundings: the mean of squares from an fp64 sum (exact
for bf16 inputs, hence independent of the summation order) rounded to fp32 once, correctly rounded fp32 square root
and division, products and sums rounded one by one (no fused multiply-adds), bf16 rounding between the normalisation
and the rotation."""
import numpy as np
import pytest
import torch

from flame_amd import workloads as W

pytestmark = pytest.mark.gpu


def _dev_bits(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16).cuda()


def _check(oracle, B, N, H, D, weight, tables, norm=True, strided=False):
    from flame_amd import capi
    print(f"[input prep] B={B} N={N} H={H} D={D} weight={weight} tables={tables} norm={norm} strided={strided}", flush=True)
    x = W.f32_to_bf16_bits(W.normal_f32(21, 0, B * N * H * D).reshape(B, N, H, D) * np.float32(1.7))
    w = W.f32_to_bf16_bits(np.linspace(0.5, 1.5, D).astype(np.float32)) if weight else None
    cos = sin = None
    if tables:
        ang = (np.arange(N, dtype=np.float64)[:, None] * 10000.0 ** (-np.arange(D // 2) / (D // 2))[None, :])
        cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        if tables == "bf16":
            cos, sin = W.f32_to_bf16_bits(cos), W.f32_to_bf16_bits(sin)
    xd = _dev_bits(x)
    if strided:      # the H dim sliced out of a wider projection output, e.g. fused QKV
        wide = torch.zeros((B, N, 3 * H, D), dtype=torch.bfloat16, device="cuda")
        wide[:, :, H:2 * H] = xd
        xd = wide[:, :, H:2 * H]
    cd = sd = None
    if tables == "f32":
        cd, sd = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    elif tables == "bf16":
        cd, sd = _dev_bits(cos), _dev_bits(sin)
    got = capi.prep_rmsnorm_rope(xd, _dev_bits(w) if weight else None, cd, sd, eps=1e-6, apply_norm=norm)
    torch.cuda.synchronize()
    got = got.view(torch.int16).cpu().numpy().view(np.uint16)
    cf = W.bf16_bits_to_f32(cos) if tables == "bf16" else cos
    sf = W.bf16_bits_to_f32(sin) if tables == "bf16" else sin
    ref = oracle.prep_rmsnorm_rope(x, w, cf, sf, eps=1e-6, apply_norm=norm)
    assert got.shape == ref.shape == (B, H, N, D)
    same = float(np.mean(got == ref))
    if same != 1.0:
        gf, rf = W.bf16_bits_to_f32(got), W.bf16_bits_to_f32(ref)
        bad = np.argwhere(got != ref)
        print(f"      {bad.shape[0]} of {got.size} outputs differ, first at {bad[0].tolist()}: {gf[tuple(bad[0])]} vs {rf[tuple(bad[0])]}", flush=True)
    assert same == 1.0, same
    return same


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("tables", [None, "f32", "bf16"])
def test_prep_small(oracle, D, tables):
    _check(oracle, 2, 37, 3, D, weight=True, tables=tables)


def test_prep_rope_only_is_bit_exact(oracle):
    assert _check(oracle, 1, 50, 4, 128, weight=False, tables="f32", norm=False) == 1.0


def test_prep_strided_input_and_no_weight(oracle):
    _check(oracle, 2, 33, 4, 128, weight=False, tables="f32", strided=True)


def test_prep_joint_attention_shape(oracle):
    # the text + image token count of the headline configuration, a few heads
    _check(oracle, 1, 4608, 4, 128, weight=True, tables="f32")


def test_prep_rejects_bad_arguments():
    from flame_amd import capi
    x = torch.zeros((1, 8, 2, 96), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(capi.FlameAttnError):
        capi.prep_rmsnorm_rope(x)                      # head dim 96 unsupported
