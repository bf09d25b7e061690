"""Helpers shared by the GPU parity tests: numpy bf16 bit patterns <-> torch device tensors."""
import numpy as np
import torch


def to_dev(bits: np.ndarray) -> torch.Tensor:
    """uint16 bf16 bit patterns -> bf16 tensor on cuda:0."""
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).cuda()


def to_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().contiguous().cpu().view(torch.int16).numpy().view(np.uint16)


def to_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


# north-star tolerances against the naive fp32-accumulated reference
TOL_MAX_ABS = 2e-2
TOL_REL_L2 = 1e-2
TOL_LSE = 1e-3


def bf16_ulp(x: np.ndarray) -> np.ndarray:
    """Spacing of bf16 numbers at magnitude |x| (8 significand bits)."""
    ax = np.maximum(np.abs(np.asarray(x, np.float64)), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(ax)) - 7)


def assert_close_bf16(oracle, name, got_f32, ref_bits, ref_f32, max_abs=TOL_MAX_ABS, stragglers=0):
    """The parity bar for a bf16 output tensor (max_abs: the flat bound, the north-star 2e-2 unless a test states why
    its quantities are scaled; stragglers: how many elements of the tensor may miss the max-abs bar below, by less
    than a factor of two, in a test that states why: their count, errors and magnitudes are printed).

    * relative L2 <= 1e-2 against the oracle's un-rounded fp32 values;
    * max-abs <= 2e-2 against both the un-rounded fp32 values and the oracle's bf16-rounded values,
      except that where one bf16 ulp is itself larger than that bound (|x| >= 4: ulp 3.1e-2) a single
      ulp is allowed: a bf16 output cannot be closer than half an ulp to an arbitrary fp32 value, and
      two correct roundings of fp32 values a hair apart may legitimately land one ulp apart.
    """
    ref_b = oracle.bf16_to_f32(ref_bits).reshape(got_f32.shape)
    ref_f = ref_f32.reshape(got_f32.shape)
    ma_f, rl_f = oracle.max_abs(got_f32, ref_f), oracle.rel_l2(got_f32, ref_f)
    diff_b = np.abs(got_f32.astype(np.float64) - ref_b.astype(np.float64))
    ma_b = float(diff_b.max()) if diff_b.size else 0.0
    diff_f = np.abs(got_f32.astype(np.float64) - ref_f.astype(np.float64))
    # elements that pass only through the one-ulp allowance (their error exceeds the flat 2e-2)
    n_ulp = int(np.count_nonzero((diff_f > max_abs) | (diff_b > max_abs)))
    print(f"      {name}: vs fp32 oracle max_abs={ma_f:.3e} rel_l2={rl_f:.3e}; vs bf16 oracle max_abs={ma_b:.3e} "
          f"(|ref|max={np.abs(ref_f).max():.2f}; {n_ulp} of {diff_f.size} elements needed the one-ulp allowance "
          f"for |x| >= 4)", flush=True)
    assert np.all(np.isfinite(got_f32)), name
    assert rl_f <= TOL_REL_L2, name
    bad = (diff_f > np.maximum(max_abs, bf16_ulp(ref_f))) | (diff_b > np.maximum(max_abs, bf16_ulp(ref_b)))
    n_bad = int(np.count_nonzero(bad))
    if n_bad and stragglers:
        print(f"      {name}: {n_bad} of {diff_f.size} elements miss the max-abs bar (allowed here: {stragglers}): errors "
              f"{np.round(diff_f[bad], 4).tolist()[:8]} at reference values {np.round(ref_f[bad], 3).tolist()[:8]}", flush=True)
        assert n_bad <= stragglers, name
        assert np.all(diff_f[bad] <= 2 * np.maximum(max_abs, bf16_ulp(ref_f[bad]))), name
    else:
        assert n_bad == 0, name
    return ma_f, rl_f
