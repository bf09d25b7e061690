"""The element-wise tile primitives under the reference's names, through the C ABI, against the CPU oracle:
masks and dropout bit-exact, the exponential / logarithm ones within fp32 and bf16 rounding.  Shapes cover the
vector paths (row length a multiple of 4 or 8, aligned base), the element-wise paths (odd lengths, offset
base), one-element and empty tiles, and a tile of the production row length."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1, 1), (2, 3, 5), (3, 17, 29), (2, 33, 64), (4, 64, 128), (1, 8, 4608), (2, 5, 72)]


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _offset_view(t, elems=1):
    """The same values at a base that is not 16-byte aligned."""
    buf = torch.empty(t.numel() + elems, dtype=t.dtype, device=t.device)
    v = buf[elems:].view(t.shape)
    v.copy_(t)
    return v


@pytest.mark.parametrize("shape", [(1, 2, 3, 4), (2, 3, 17, 29), (1, 2, 64, 128), (2, 1, 5, 72)])
@pytest.mark.parametrize("offsets", [(0, 0), (5, 9), (40, 3), (0, 1000), (1000, 0)])
def test_causal_and_keep_masks_bit_exact(oracle, shape, offsets):
    from flame_amd import capi
    print(f"[tile] masks {shape} offsets {offsets}", flush=True)
    rng = np.random.default_rng(hash((shape, offsets)) % 2 ** 32)
    x = rng.normal(size=shape).astype(np.float32)
    for view in (lambda t: t, _offset_view):
        got = capi.tile_causal_mask(view(_dev(x)), *offsets)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), oracle.tile_causal_mask(x.copy(), *offsets))
    m = rng.integers(0, 3, size=shape).astype(np.uint8)
    m[..., : shape[-1] // 2] = np.where(rng.random(m[..., : shape[-1] // 2].shape) < 0.8, 1, m[..., : shape[-1] // 2])
    for view in (lambda t: t, _offset_view):
        got = capi.tile_attn_mask(view(_dev(x)), view(_dev(m)))
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), oracle.tile_attn_mask(x.copy(), m))
    zeros = np.zeros(shape, np.uint8)
    assert torch.all(capi.tile_attn_mask(_dev(x), _dev(zeros)) == -1.0e9)


@pytest.mark.parametrize("shape", SHAPES)
def test_additive_tile_mask_bit_exact(oracle, shape):
    from flame_amd import capi
    BH, q_t, k_t = shape
    print(f"[tile] add_mask {shape}", flush=True)
    rng = np.random.default_rng(BH * 1000 + q_t * 10 + k_t)
    x = rng.normal(size=shape).astype(np.float32)
    x[0, 0, 0] = -0.0                                    # -0 + 0 = +0: the write may not be skipped
    k_total, k0, q0 = k_t + 11, 7, k_t // 2
    b3 = rng.integers(0, 2, size=shape).astype(np.uint8)
    b2 = rng.integers(0, 2, size=(BH, k_total)).astype(np.uint8)
    a3 = rng.normal(size=shape).astype(np.float32)
    a2 = rng.normal(size=(BH, k_total)).astype(np.float32)
    cases = [dict(user_bool=b3, user_add=a3, bool_rank=3, add_rank=3, zero_is_mask=True, causal=False),
             dict(user_bool=b2, user_add=a2, bool_rank=2, add_rank=2, zero_is_mask=False, causal=True),
             dict(user_bool=b3, user_add=None, bool_rank=3, zero_is_mask=False, causal=True),
             dict(user_bool=None, user_add=a2, add_rank=2, causal=False),
             dict(user_bool=None, user_add=None, causal=True),
             dict(user_bool=None, user_add=None, causal=False),
             dict(user_bool=b3, user_add=a3, bool_rank=1, add_rank=0, causal=False)]
    for c in cases:
        want = oracle.tile_add_mask(x.copy(), q_abs_start=q0, k_abs_start=k0, k_total=k_total, **c)
        dc = {k: (_dev(v) if isinstance(v, np.ndarray) else v) for k, v in c.items()}
        for view in (lambda t: t, _offset_view):
            got = capi.tile_add_mask(view(_dev(x)), q_abs_start=q0, k_abs_start=k0, k_total=k_total, **dc)
            torch.cuda.synchronize()
            g = got.cpu().numpy()
            assert np.array_equal(g.view(np.uint32), want.view(np.uint32)), c


@pytest.mark.parametrize("shape", SHAPES)
def test_lse_softmax_and_merge(oracle, shape):
    from flame_amd import capi
    BH, q_t, k_t = shape
    print(f"[tile] lse/softmax {shape}", flush=True)
    rng = np.random.default_rng(BH * 77 + q_t * 5 + k_t)
    x = (rng.normal(size=shape) * 4).astype(np.float32)
    if q_t > 1:
        x[0, 1, :] = -1.0e30                             # a row the reference's masks have excluded whole
    if k_t > 2:
        x[0, 0, 1] = -np.inf
    want_lse = oracle.tile_lse_from_logits(x)
    for view in (lambda t: t, _offset_view):
        lse = capi.tile_lse_from_logits(view(_dev(x)))
        torch.cuda.synchronize()
        err = np.abs(lse.cpu().numpy() - want_lse)
        assert np.all(err <= 1e-5 * np.maximum(1.0, np.abs(want_lse))), err.max()
    # probabilities from the oracle's own lse, so that only this kernel's arithmetic is compared
    want_bits, want_p32 = oracle.tile_softmax_from_lse(x, want_lse)
    for view in (lambda t: t, _offset_view):
        probs = capi.tile_softmax_from_lse(view(_dev(x)), _dev(want_lse))
        torch.cuda.synchronize()
        got = probs.float().cpu().numpy()
        # bf16 rounding of a value within 2e-6 relative of the oracle's: at most one bf16 step apart, and only
        # where the fp32 value sits at a rounding boundary
        ref = oracle.bf16_to_f32(want_bits)
        assert np.all(np.abs(got - ref) <= np.maximum(ref, 1e-30) * 2.0 ** -7)
        assert np.mean(got != ref) <= 0.01
        assert np.abs(got - want_p32).max() <= 2.0 ** -8
    other = (rng.normal(size=(BH, q_t)) * 3).astype(np.float32)
    if q_t > 1:
        other[0, 1] = -np.inf
    want = oracle.tile_lse_merge(want_lse.copy(), other)
    got = capi.tile_lse_merge(_dev(want_lse), _dev(other))
    torch.cuda.synchronize()
    assert np.all(np.abs(got.cpu().numpy() - want) <= 1e-5 * np.maximum(1.0, np.abs(want)))
    ninf = np.full((BH, q_t), -np.inf, np.float32)
    assert torch.all(capi.tile_lse_merge(_dev(ninf), _dev(ninf)) == -np.inf)


@pytest.mark.parametrize("shape", SHAPES + [(3, 4, 0), (0, 4, 8)])
def test_dropout_bit_exact(oracle, shape):
    from flame_amd import capi
    BH, q_t, k_t = shape
    print(f"[tile] dropout {shape}", flush=True)
    rng = np.random.default_rng(BH * 31 + q_t * 3 + k_t)
    x = oracle.f32_to_bf16(rng.random(size=shape).astype(np.float32))
    for p, seed in ((0.1, 1), (0.3, 2024), (0.5, 0x9E3779B97F4A7C15), (0.0, 5), (1.0, 5)):
        want = oracle.tile_dropout(x.copy(), p, seed)
        for view in (lambda t: t, _offset_view):
            t = view(_dev(x).view(torch.bfloat16))
            got = capi.tile_dropout(t, p, seed)
            torch.cuda.synchronize()
            assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want), (p, seed)


def test_empty_tiles_and_bad_arguments():
    from flame_amd import capi
    import ctypes
    lib = capi.lib()
    null = ctypes.c_void_p(0)
    assert lib.flame_apply_causal_mask_fp32(null, 0, 1, 4, 4, 0, 0, null) == 0
    assert lib.flame_apply_causal_mask_fp32(null, 1, 1, 4, 4, 0, 0, null) == 1
    assert lib.flame_apply_causal_mask_fp32(null, 1, 1, -4, 4, 0, 0, null) == 1
    assert lib.flame_sdpa_lse_merge_rows(null, null, 2, 0, null) == 0
    assert lib.flame_sdpa_dropout_bf16_inplace(null, ctypes.c_float(0.5), ctypes.c_uint64(1), 1, 1, 1, null) == 1
    out = torch.zeros((2, 3), dtype=torch.float32, device="cuda")
    assert lib.flame_sdpa_lse_from_logits_tile(null, ctypes.c_void_p(out.data_ptr()), 2, 3, 0, null) == 0
    torch.cuda.synchronize()
    assert torch.all(out == -np.inf)                     # a row without elements
