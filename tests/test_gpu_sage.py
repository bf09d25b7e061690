"""GPU parity of the SageAttention int8-QK path: quantised tensors and scales bit-exact against the
CPU oracle, output cosine >= 0.999 against the bf16 kernel on the same inputs."""
import math

import numpy as np
import pytest
import torch

from flame_amd import workloads as W
from tests.gpu_util import to_dev, to_f32

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
    ro, rlse = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale)
    # same quantised operands on both sides: only P->bf16 and accumulation order differ
    assert oracle.max_abs(to_f32(o), oracle.bf16_to_f32(ro)) <= 2e-2
    assert oracle.rel_l2(to_f32(o), oracle.bf16_to_f32(ro)) <= 1e-2
    assert oracle.max_abs(lse.cpu().numpy().reshape(rlse.shape), rlse) <= 1e-3
    cos = oracle.cosine(to_f32(o), to_f32(o_bf16))
    print(f"      cosine vs bf16 path = {cos:.6f}", flush=True)
    assert cos >= 0.999


def test_sage_causal_and_key_length(oracle):
    from flame_amd import capi
    w = W.config5(B=2, H=2, S=200, D=64)
    q, k, v = (to_dev(t) for t in (w.q, w.k, w.v))
    qz = capi.sage_quant(q, k)
    o_c = capi.sage_fwd(qz, v, w.scale, causal=True)
    ref_c, _ = capi.attn_fwd(q, k, v, w.scale, causal=True)
    assert oracle.cosine(to_f32(o_c), to_f32(ref_c)) >= 0.999
    kvl = torch.tensor([200, 77], dtype=torch.int32, device="cuda")
    o_l = capi.sage_fwd(qz, v, w.scale, kv_len=kvl)
    ref_l, _ = capi.attn_fwd(q, k, v, w.scale, kv_len=kvl)
    assert oracle.cosine(to_f32(o_l), to_f32(ref_l)) >= 0.999


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
    # oracle parity of the int8 forward on one head
    ro, _ = oracle.sage_fwd(ref["qi8"], ref["ki8"], ref["sq"], ref["sk"], w.v, w.scale, heads=(5, 6))
    assert oracle.rel_l2(a.reshape(48, 4608, 128)[5], oracle.bf16_to_f32(ro).reshape(48, 4608, 128)[5]) <= 1e-2
