"""Python-level counterparts of the reference's PyO3 functions for this path
(src/python/functional.rs:187-241 `sdpa`, src/python/nn.rs:390-428 `scaled_dot_product_attention`),
on torch tensors that live on the GPU.  Both are differentiable: the forward saves O and the per-row
log-sum-exp only, the backward recomputes the probabilities tile by tile in the HIP kernels.

Nothing here falls back to torch arithmetic: without the HIP library the calls raise.
"""
from __future__ import annotations

import math

import torch

from . import capi


class _Sdpa(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask_u8, causal, scale):
        # the fused kernels where they serve the shape, else the materialised path (any head dim, masks above 128),
        # as the reference's dispatch does (src/sdpa.rs:483-587); both save O and the log-sum-exp only
        ctx.materialised = False
        try:
            o, lse = capi.attn_fwd(q, k, v, scale, causal=causal, mask=mask_u8)
        except capi.FlameAttnError as e:
            if e.code != capi.ERR_UNSUPPORTED:
                raise
            o, lse = capi.attn_fwd_materialised(q, k, v, scale, causal=causal, mask=mask_u8)
            ctx.materialised = True
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.mask_u8, ctx.causal, ctx.scale = mask_u8, causal, scale
        return o

    @staticmethod
    def backward(ctx, grad_out):
        q, k, v, o, lse = ctx.saved_tensors
        g = grad_out.to(torch.bfloat16)
        if g.stride(-1) != 1 or any(s % 8 for s in g.stride()[:-1]):
            g = g.contiguous()
        if not ctx.materialised:
            try:
                return (*capi.attn_bwd(q, k, v, o, g, lse, ctx.scale, causal=ctx.causal, mask=ctx.mask_u8), None, None, None)
            except capi.FlameAttnError as e:         # a head dim the fused forward serves and the fused backward does not
                if e.code != capi.ERR_UNSUPPORTED:
                    raise
        dq, dk, dv = capi.attn_bwd_materialised(q, k, v, o, g, lse, ctx.scale, causal=ctx.causal, mask=ctx.mask_u8)
        return dq, dk, dv, None, None, None


def _as_bf16_view(t: torch.Tensor) -> torch.Tensor:
    t = t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)     # promote_bf16 of the reference
    if t.shape[-1] % 8 == 0 and (t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or (t.storage_offset() % 8)):
        t = t.contiguous()
    elif t.stride(-1) != 1:
        t = t.contiguous()
    return t


def sdpa(q, k, v, attn_mask=None, is_causal=None, scale=None):
    """Scaled dot-product attention on [B,H,S,D] tensors.

    attn_mask: optional binary keep-mask broadcastable as [B|1, H|1, Sq, Sk] (values >= 0.5 attend; the
    reference's public mask convention, src/sdpa.rs:458-470).  With is_causal=True the mask argument is
    ignored, as in the reference, and the causal structure is applied natively (no mask tensor is built).
    Inputs of another dtype are promoted to bf16 and the result is cast back."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("SDPA expects 4-D input [B, H, S, D]")
    orig = q.dtype
    causal = bool(is_causal) if is_causal is not None else False
    qb, kb, vb = _as_bf16_view(q), _as_bf16_view(k), _as_bf16_view(v)
    mask_u8 = None
    if not causal and attn_mask is not None:
        if attn_mask.dim() != 4:
            raise ValueError("mask must be 4D [B,H,Q,K]")
        mask_u8 = attn_mask if attn_mask.dtype == torch.uint8 else (attn_mask.float() >= 0.5).to(torch.uint8)
    sc = float(scale) if scale is not None else 1.0 / math.sqrt(q.shape[-1])
    out = _Sdpa.apply(qb, kb, vb, mask_u8, causal, sc)
    return out if orig == torch.bfloat16 else out.to(orig)


def scaled_dot_product_attention(q, k, v, is_causal=None):
    """nn.scaled_dot_product_attention of the reference: bf16 [B,H,S,D], scale 1/sqrt(D), optional causal."""
    if q.dim() != 4:
        raise ValueError("SDPA expects 4-D input [B, H, S, D]")
    return sdpa(q, k, v, None, is_causal)


def sdpa_with_bias(q, k, v, bias=None, scale=None):
    """attention::sdpa_with_bias: softmax(scale * Q K^T + bias) V with an additive float bias (inference only)."""
    if bias is None:
        return sdpa(q, k, v, scale=scale)
    orig = q.dtype
    sc = float(scale) if scale is not None else 1.0 / math.sqrt(q.shape[-1])
    b = bias if bias.dtype in (torch.float32, torch.bfloat16) else bias.float()
    o, _ = capi.attn_fwd_bias(_as_bf16_view(q), _as_bf16_view(k), _as_bf16_view(v), sc, b, want_lse=False)
    return o if orig == torch.bfloat16 else o.to(orig)
