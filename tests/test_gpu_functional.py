"""The Python-level sdpa() against a plain PyTorch fp32 reference of the same op (torch arithmetic on
the GPU, materialised scores), forward and backward through torch.autograd."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ref(q, k, v, mask=None, causal=False, bias=None, scale=None):
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    sc = scale if scale is not None else 1.0 / math.sqrt(q.shape[-1])
    s = torch.einsum("bhqd,bhkd->bhqk", qf, kf) * sc
    if bias is not None:
        s = s + bias.float()
    if causal:
        i = torch.arange(q.shape[2], device=q.device)[:, None]
        j = torch.arange(k.shape[2], device=q.device)[None, :]
        s = s.masked_fill(j > i, float("-inf"))
    if mask is not None:
        s = s.masked_fill(mask.float() < 0.5, float("-inf"))
    o = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, dim=-1), vf)
    return o, (qf, kf, vf)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128, 20, 264])      # 20 and 264 (with its mask and its backward): the materialised path
def test_sdpa_forward_backward_vs_torch_fp32(causal, D):
    from flame_amd import functional as F
    torch.manual_seed(3)
    B, H, Sq, Sk = 2, 3, 150, 150 if causal else 233
    print(f"[functional] causal={causal} D={D}", flush=True)
    q, k, v = (torch.randn(B, H, n, D, device="cuda").to(torch.bfloat16).requires_grad_(True) for n in (Sq, Sk, Sk))
    mask = None if causal else (torch.rand(B, 1, Sq, Sk, device="cuda") < 0.7)
    if mask is not None:
        mask[..., 0] = True
    o = F.sdpa(q, k, v, attn_mask=None if mask is None else mask.to(torch.bfloat16), is_causal=causal)
    g = torch.randn_like(o)
    o.backward(g)
    ro, (qf, kf, vf) = _ref(q, k, v, mask=mask, causal=causal)
    ro.backward(g.float())
    assert (o.float() - ro).abs().max().item() <= 2e-2
    for name, a, b in (("dq", q.grad, qf.grad), ("dk", k.grad, kf.grad), ("dv", v.grad, vf.grad)):
        err = (a.float() - b).abs()
        tol = torch.maximum(torch.full_like(b, 2e-2), torch.pow(2.0, torch.floor(torch.log2(b.abs().clamp_min(1e-30))) - 7))
        assert bool((err <= tol).all()), (name, err.max().item())
        assert (err.pow(2).sum().sqrt() / b.pow(2).sum().sqrt()).item() <= 1e-2, name


def test_fp32_inputs_are_promoted_and_cast_back():
    from flame_amd import functional as F
    q, k, v = (torch.randn(1, 2, 70, 64, device="cuda") for _ in range(3))
    o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert o.dtype == torch.float32 and o.shape == q.shape
    ro, _ = _ref(q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16), causal=True)
    assert (o - ro).abs().max().item() <= 2e-2


def test_sdpa_with_bias_vs_torch_fp32():
    from flame_amd import functional as F
    torch.manual_seed(4)
    q, k, v = (torch.randn(2, 4, n, 64, device="cuda").to(torch.bfloat16) for n in (90, 120, 120))
    bias = torch.randn(1, 4, 90, 120, device="cuda")
    o = F.sdpa_with_bias(q, k, v, bias, scale=1.0)            # T5 style: unscaled logits
    ro, _ = _ref(q, k, v, bias=bias, scale=1.0)
    assert (o.float() - ro).abs().max().item() <= 2e-2


def test_rank_check():
    from flame_amd import functional as F
    with pytest.raises(ValueError):
        F.sdpa(torch.zeros(2, 3, 4, device="cuda"), torch.zeros(2, 3, 4, device="cuda"), torch.zeros(2, 3, 4, device="cuda"))
