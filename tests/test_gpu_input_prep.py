"""GPU parity of the fused input preparation (RMS-norm + RoPE + layout change) against the oracle.

The kernel follows the same roundings as the oracle; what may differ is the last fp32 bit of the
mean of squares (summation order) and of rsqrt, which can move a normalised value across a bf16
rounding boundary; the rotation then spreads that one step over both outputs of the pair.  Bar: at
least 99.9 % of the outputs bit-identical, every output within one bf16 step of its own plus 1.5
steps of the larger normalised value of its pair; without the normalisation: bit-identical."""
import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import bf16_ulp

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
    gf, rf = W.bf16_bits_to_f32(got), W.bf16_bits_to_f32(ref)
    bound = bf16_ulp(rf)
    if norm and tables:
        nf = np.abs(W.bf16_bits_to_f32(oracle.prep_rmsnorm_rope(x, w, None, None, eps=1e-6)))
        pair = np.maximum(nf[..., 0::2], nf[..., 1::2])
        bound = bound + 1.5 * np.repeat(bf16_ulp(pair), 2, axis=-1)
    assert np.all(np.abs(gf - rf) <= bound), float(np.max(np.abs(gf - rf) / bound))
    same = float(np.mean(got == ref))
    assert same >= 0.999, same
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
