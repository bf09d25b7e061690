"""The BF16 <-> FP8 E4M3 pair of the activation offload pool on the GPU (flame_bf16_to_fp8 / flame_fp8_to_bf16,
reference src/cuda/fp8_quant.cu, src/cuda/fp8_dequant.cu) against the CPU oracle, bit for bit: every bf16 input and
every code at several scales, vector and scalar paths (aligned and misaligned pointers, lengths around multiples of
16), a saved-activation sized tensor, and the round trip through both kernels."""
import numpy as np
import pytest
import torch

from flame_amd import workloads as W

pytestmark = pytest.mark.gpu

POOL_SCALE = float(np.float32(8.0 / 448.0))                 # src/activation_offload.rs:548-549
POOL_INV = float(np.float32(1.0) / np.float32(POOL_SCALE))


def _dev_bits(bits):
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def _host_bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("inv_scale", [1.0, POOL_INV, float(np.float32(1.0 / 0.37)), 2.0 ** -100, 2.0 ** 90, 1e-40, -3.0])
def test_every_bf16_input_encodes_as_the_oracle_says(oracle, inv_scale):
    from flame_amd import capi
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = capi.bf16_to_fp8(_dev_bits(bits), inv_scale).cpu().numpy()
    assert np.array_equal(got, oracle.bf16_to_fp8(bits, inv_scale))


@pytest.mark.parametrize("scale", [1.0, POOL_SCALE, 0.37, 3.0e38, 2.0 ** -120, 1e-40, -0.5])
def test_every_code_decodes_as_the_oracle_says(oracle, scale):
    from flame_amd import capi
    codes = np.tile(np.arange(256, dtype=np.uint8), 3)       # 768 elements: vector path
    got = _host_bits(capi.fp8_to_bf16(torch.from_numpy(codes).cuda(), scale))
    assert np.array_equal(got, oracle.fp8_to_bf16(codes, scale))


@pytest.mark.parametrize("n", [1, 15, 16, 17, 31, 4096 + 5, 100003])
@pytest.mark.parametrize("shift", [0, 1, 8])
def test_lengths_and_alignments(oracle, n, shift):
    """shift: elements by which both tensors start past a 16-byte boundary (1 -> the scalar path)."""
    from flame_amd import capi
    x = W.f32_to_bf16_bits(W.normal_f32(7100 + n, shift, n) * np.float32(1.7))
    xd = torch.zeros(n + 64, dtype=torch.bfloat16, device="cuda")
    xd[shift:shift + n] = _dev_bits(x)
    cd = torch.full((n + 64,), 0xAA, dtype=torch.uint8, device="cuda")
    capi.bf16_to_fp8(xd[shift:shift + n], POOL_INV, out=cd[shift:shift + n])
    want = oracle.bf16_to_fp8(x, POOL_INV)
    got = cd.cpu().numpy()
    assert np.array_equal(got[shift:shift + n], want)
    assert np.all(got[:shift] == 0xAA) and np.all(got[shift + n:] == 0xAA)          # nothing written outside
    bd = torch.full((n + 64,), -7.0, dtype=torch.bfloat16, device="cuda")
    capi.fp8_to_bf16(cd[shift:shift + n], POOL_SCALE, out=bd[shift:shift + n])
    gb = _host_bits(bd)
    assert np.array_equal(gb[shift:shift + n], oracle.fp8_to_bf16(want, POOL_SCALE))
    assert np.all(gb[:shift] == 0xC0E0) and np.all(gb[shift + n:] == 0xC0E0)


def test_saved_attention_output_round_trip(oracle):
    """A saved O of the headline shape (1 x 24 x 4608 x 128, attention outputs of unit-variance V): both kernels
    bit-exact against the oracle, and the round-trip error of the format: relative 2^-4 per element at most,
    about 2 % in relative L2."""
    from flame_amd import capi
    n = 24 * 4608 * 128
    x = W.f32_to_bf16_bits(W.normal_f32(7200, 0, n) * np.float32(0.6))
    xd = _dev_bits(x)
    codes = capi.bf16_to_fp8(xd, POOL_INV)
    back = capi.fp8_to_bf16(codes, POOL_SCALE)
    torch.cuda.synchronize()
    want_codes = oracle.bf16_to_fp8(x, POOL_INV)
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(_host_bits(back), oracle.fp8_to_bf16(want_codes, POOL_SCALE))
    ref, got = oracle.bf16_to_f32(x), back.float().cpu().numpy()
    err = np.abs(got - ref)
    assert np.all(err <= np.abs(ref) / 16 * 1.01 + 2.0 ** -9 * POOL_SCALE * 1.01)
    assert oracle.rel_l2(got, ref) < 0.03


def test_empty_and_null_arguments():
    import ctypes
    from flame_amd import capi
    lib = capi.lib()
    z = ctypes.c_void_p(0)
    assert lib.flame_bf16_to_fp8(z, z, ctypes.c_float(1.0), ctypes.c_size_t(0), z) == 0       # n = 0: nothing to do
    assert lib.flame_fp8_to_bf16(z, z, ctypes.c_float(1.0), ctypes.c_size_t(0), z) == 0
    assert lib.flame_bf16_to_fp8(z, z, ctypes.c_float(1.0), ctypes.c_size_t(8), z) != 0
    assert lib.flame_fp8_to_bf16(z, z, ctypes.c_float(1.0), ctypes.c_size_t(8), z) != 0
