"""ctypes binding of ``libflame_attn_hip.so`` (the C ABI declared in ``include/flame_attn.h``).

Tensors are torch CUDA(HIP) tensors used purely as device-memory handles: the library receives raw
pointers, element strides and the current HIP stream.  There is no CPU path: if the shared library
is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FLAME_ATTN_LIB") or os.path.join(_HERE, "lib", "libflame_attn_hip.so")
_lib = None

OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_TOO_LARGE = 0, -1, -2, -3


class FlameAttnError(RuntimeError):
    def __init__(self, fn: str, code: int):
        self.code = code
        kind = {ERR_INVALID: "invalid argument", ERR_UNSUPPORTED: "unsupported",
                ERR_TOO_LARGE: "too many query rows for the fixed scratch"}.get(code, "HIP error")
        super().__init__(f"{fn} failed: {kind} ({code})")


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m flame_amd.build` (hipcc, gfx950)")
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib


def _i64x4(vals):
    return (ctypes.c_int64 * 4)(*[int(v) for v in vals])


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _mask_strides(mask, B, H, Sq, Sk):
    if mask is None:
        return None
    assert mask.dtype == torch.uint8 and mask.dim() == 4
    full = (B, H, Sq, Sk)
    st = []
    for ax in range(4):
        assert mask.shape[ax] in (1, full[ax]), "mask is not broadcastable to [B,H,Sq,Sk]"
        st.append(0 if (mask.shape[ax] == 1 and full[ax] != 1) else mask.stride(ax))
    return _i64x4(st)


def fwd_workspace_bytes(B, H, Sq, Sk, D) -> int:
    """Bytes of workspace with which flame_attn_fwd_ws_bf16 splits the keys of a small problem at a head dim above
    128 over workgroups (0 where it would not split)."""
    f = lib().flame_attn_fwd_workspace_bytes
    f.restype = ctypes.c_size_t
    return int(f(B, H, Sq, Sk, D))


def attn_fwd(q, k, v, scale, causal=False, kv_len=None, mask=None, want_lse=True, out=None, lse_out=None, workspace=None):
    """O, LSE = flame_attn_fwd_bf16(...).  q [B,H,Sq,D], k/v [B,H,Sk,D] bf16, D stride 1.
    `workspace` (uint8 device tensor): flame_attn_fwd_ws_bf16 instead, which may use it."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    o = torch.empty((B, H, Sq, D), dtype=torch.bfloat16, device=q.device) if out is None else out
    lse = lse_out if lse_out is not None else (torch.empty((B * H, Sq), dtype=torch.float32, device=q.device) if want_lse else None)
    ms = _mask_strides(mask, B, H, Sq, Sk)
    args = (_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, H, Sq, Sk, D, ctypes.c_float(scale),
            _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
            *(ctypes.c_int64(0) for _ in range(5)),
            int(bool(causal)), _ptr(kv_len), _ptr(mask), ms)
    if workspace is None:
        fn, rc = "flame_attn_fwd_bf16", lib().flame_attn_fwd_bf16(*args, _stream())
    else:
        fn, rc = "flame_attn_fwd_ws_bf16", lib().flame_attn_fwd_ws_bf16(
            *args, _ptr(workspace), ctypes.c_size_t(workspace.numel()), _stream())
    if rc != 0:
        raise FlameAttnError(fn, rc)
    return o, lse


def attn_fwd_bias(q, k, v, scale, bias, mask=None, want_lse=True):
    """softmax(scale * Q K^T + bias) V.  bias: fp32 or bf16 [B|1, H|1, Sq, Sk] (inference only)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    assert bias.dim() == 4 and bias.dtype in (torch.float32, torch.bfloat16)
    full = (B, H, Sq, Sk)
    bst = []
    for ax in range(4):
        assert bias.shape[ax] in (1, full[ax]), "bias is not broadcastable to [B,H,Sq,Sk]"
        bst.append(0 if (bias.shape[ax] == 1 and full[ax] != 1) else bias.stride(ax))
    o = torch.empty((B, H, Sq, D), dtype=torch.bfloat16, device=q.device)
    lse = torch.empty((B * H, Sq), dtype=torch.float32, device=q.device) if want_lse else None
    rc = lib().flame_attn_fwd_bias_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, H, Sq, Sk, D, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        *(ctypes.c_int64(0) for _ in range(5)),
        _ptr(bias), 1 if bias.dtype == torch.float32 else 0, _i64x4(bst),
        _ptr(mask), _mask_strides(mask, B, H, Sq, Sk), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_fwd_bias_bf16", rc)
    return o, lse


def bwd_workspace_bytes(B, H, Sq, D) -> int:
    f = lib().flame_attn_bwd_workspace_bytes
    f.restype = ctypes.c_size_t
    return int(f(B, H, Sq, D))


def attn_bwd(q, k, v, o, do, lse, scale, causal=False, kv_len=None, mask=None, workspace=None, grads=None):
    """dQ, dK, dV = flame_attn_bwd_bf16(...).  `workspace`: uint8 device tensor of at least
    bwd_workspace_bytes(...) bytes (allocated here when omitted)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    need = bwd_workspace_bytes(B, H, Sq, D)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    if grads is None:
        dq = torch.empty((B, H, Sq, D), dtype=torch.bfloat16, device=q.device)
        dk = torch.empty((B, H, Sk, D), dtype=torch.bfloat16, device=q.device)
        dv = torch.empty((B, H, Sk, D), dtype=torch.bfloat16, device=q.device)
    else:
        dq, dk, dv = grads
    ms = _mask_strides(mask, B, H, Sq, Sk)
    rc = lib().flame_attn_bwd_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
        B, H, Sq, Sk, D, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        _i64x4(do.stride()), _i64x4(dq.stride()), _i64x4(dk.stride()), _i64x4(dv.stride()),
        *(ctypes.c_int64(0) for _ in range(9)),
        int(bool(causal)), _ptr(kv_len), _ptr(mask), ms,
        _ptr(workspace), ctypes.c_size_t(workspace.numel()), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_bwd_bf16", rc)
    return dq, dk, dv


def attn_bwd_noalloc(q, k, v, o, do, lse, scale, grads, causal=False, kv_len=None, mask=None):
    """flame_attn_bwd_bf16_noalloc(...): the backward on the library's fixed device scratch.  The caller
    passes the gradient tensors; nothing is allocated on the way."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    dq, dk, dv = grads
    ms = _mask_strides(mask, B, H, Sq, Sk)
    rc = lib().flame_attn_bwd_bf16_noalloc(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
        B, H, Sq, Sk, D, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        _i64x4(do.stride()), _i64x4(dq.stride()), _i64x4(dk.stride()), _i64x4(dv.stride()),
        *(ctypes.c_int64(0) for _ in range(9)),
        int(bool(causal)), _ptr(kv_len), _ptr(mask), ms, _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_bwd_bf16_noalloc", rc)
    return dq, dk, dv


def cudnn_sdpa_bwd(q, k, v, o, do, stats, scale, grads=None):
    """flame_cudnn_sdpa_bwd_bf16(...): the reference-named backward (no workspace argument)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    if grads is None:
        grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    dq, dk, dv = grads
    rc = lib().flame_cudnn_sdpa_bwd_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(stats), _ptr(dq), _ptr(dk), _ptr(dv),
        B, H, Sq, Sk, D, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        _i64x4(do.stride()), _i64x4(dq.stride()), _i64x4(dk.stride()), _i64x4(dv.stride()),
        *(ctypes.c_int64(0) for _ in range(9)), _stream())
    if rc != 0:
        raise FlameAttnError("flame_cudnn_sdpa_bwd_bf16", rc)
    return dq, dk, dv


KERNEL_KINDS = ("fwd", "unused1", "bwd_dkdv", "bwd_dq", "sage_kmean", "sage_quant", "sage_fwd", "input_prep",
                "bwd_merge", "bwd_joint", "bwd_rows", "reserved11")


class _KernelTimes(ctypes.Structure):
    _fields_ = [("total_ms", ctypes.c_double * 12), ("launches", ctypes.c_int * 12)]


def profiling_enable(on: bool) -> None:
    """Bracket every kernel launch with HIP events on the launch stream (clears earlier samples)."""
    rc = lib().flame_attn_profiling_enable(int(bool(on)))
    if rc != 0:
        raise FlameAttnError("flame_attn_profiling_enable", rc)


def profiling_read() -> dict:
    """{kernel: (total_ms, launches)} since the last read; waits for the recorded events."""
    kt = _KernelTimes()
    rc = lib().flame_attn_profiling_read(ctypes.byref(kt))
    if rc != 0:
        raise FlameAttnError("flame_attn_profiling_read", rc)
    return {name: (kt.total_ms[i], kt.launches[i]) for i, name in enumerate(KERNEL_KINDS)}


def sage_row_elems(D) -> int:
    """Row length of the tensors the Sage quantiser writes for head dim D (64 up to D = 64, else 128)."""
    return 64 if D <= 64 else 128


def sage_quant(q, k, smooth_k=True, want_ks=False):
    """Per-block int8 quantisation of Q (128 rows) and mean-smoothed K (64 rows).

    Returns dict(qi8, ki8, sq, sk, kmean[, ks]): int8 [B,H,S,D], fp32 [B,H,nblk], fp32 [B,H,D]; with
    want_ks also the smoothed bf16 K that was quantised.  For head dims other than 64 and 128 the library writes
    rows of sage_row_elems(D) elements, zero beyond D: the tensors returned are the [..., :D] views of those."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    dev = q.device
    Dp = sage_row_elems(D)
    out = dict(
        qi8=torch.empty((B, H, Sq, Dp), dtype=torch.int8, device=dev)[..., :D],
        ki8=torch.empty((B, H, Sk, Dp), dtype=torch.int8, device=dev)[..., :D],
        sq=torch.empty((B, H, -(-Sq // 128)), dtype=torch.float32, device=dev),
        sk=torch.empty((B, H, -(-Sk // 64)), dtype=torch.float32, device=dev),
        kmean=torch.empty((B, H, Dp), dtype=torch.float32, device=dev)[..., :D])
    if want_ks:
        out["ks"] = torch.empty((B, H, Sk, Dp), dtype=torch.bfloat16, device=dev)[..., :D]
    rc = lib().flame_sage_quant_qk_int8_ks(
        _ptr(q), _ptr(k), B, H, Sq, Sk, D, _i64x4(q.stride()), _i64x4(k.stride()),
        ctypes.c_int64(0), ctypes.c_int64(0), int(bool(smooth_k)),
        _ptr(out["qi8"]), _ptr(out["ki8"]), _ptr(out["sq"]), _ptr(out["sk"]), _ptr(out["kmean"]),
        _ptr(out.get("ks")), _stream())
    if rc != 0:
        raise FlameAttnError("flame_sage_quant_qk_int8_ks", rc)
    return out


def sage_fwd(qz, v, scale, causal=False, kv_len=None, want_lse=False, out=None, bias=None):
    """O (and LSE) from quantised operands `qz` (the dict returned by sage_quant) and bf16 V.
    bias: additive fp32 or bf16 [B|1, H|1, Sq, Sk] on the scaled logits (-inf excludes), or None."""
    B, H, Sq, D = qz["qi8"].shape
    Sk = qz["ki8"].shape[2]
    o = torch.empty((B, H, Sq, D), dtype=torch.bfloat16, device=v.device) if out is None else out
    lse = torch.empty((B * H, Sq), dtype=torch.float32, device=v.device) if want_lse else None
    bst, bdt = None, 1
    if bias is not None:
        assert bias.dim() == 4 and bias.dtype in (torch.float32, torch.bfloat16)
        full = (B, H, Sq, Sk)
        st = []
        for ax in range(4):
            assert bias.shape[ax] in (1, full[ax]), "bias is not broadcastable to [B,H,Sq,Sk]"
            st.append(0 if (bias.shape[ax] == 1 and full[ax] != 1) else bias.stride(ax))
        bst, bdt = _i64x4(st), (1 if bias.dtype == torch.float32 else 0)
    rc = lib().flame_sage_attn_fwd_bias_int8(
        _ptr(qz["qi8"]), _ptr(qz["ki8"]), _ptr(qz["sq"]), _ptr(qz["sk"]), _ptr(v), _ptr(o), _ptr(lse),
        B, H, Sq, Sk, D, ctypes.c_float(scale), _i64x4(v.stride()), _i64x4(o.stride()),
        ctypes.c_int64(0), ctypes.c_int64(0), int(bool(causal)), _ptr(kv_len), _ptr(bias), bdt, bst, _stream())
    if rc != 0:
        raise FlameAttnError("flame_sage_attn_fwd_bias_int8", rc)
    return (o, lse) if want_lse else o


def prep_rmsnorm_rope(x_bnhd, weight=None, cos=None, sin=None, eps=1e-6, apply_norm=True, out=None):
    """Fused RMS-norm over the head dim + interleaved RoPE + [B,N,H,D] -> [B,H,N,D].

    x_bnhd: bf16 [B,N,H,D] (any B/N/H strides); weight: bf16 [D] or None; cos/sin: [N,D/2] fp32 or
    bf16, or None.  Returns a contiguous bf16 [B,H,N,D] tensor."""
    B, N, H, D = x_bnhd.shape
    xv = x_bnhd.permute(0, 2, 1, 3)                       # logical [B,H,N,D] view of the same memory
    if out is None:
        out = torch.empty((B, H, N, D), dtype=torch.bfloat16, device=x_bnhd.device)
    tdt = 0
    if cos is not None:
        if cos.dtype != sin.dtype or cos.shape != sin.shape or tuple(cos.shape) != (N, D // 2):
            raise ValueError("cos/sin must both be [N, D/2] of one dtype")
        if not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("cos/sin must be contiguous")
        tdt = 1 if cos.dtype == torch.float32 else 0
    rc = lib().flame_attn_prep_rmsnorm_rope_bf16(
        _ptr(xv), _ptr(weight) if weight is not None else None,
        _ptr(cos) if cos is not None else None, _ptr(sin) if sin is not None else None, tdt,
        _ptr(out), B, H, N, D, ctypes.c_float(eps), int(bool(apply_norm)),
        _i64x4(xv.stride()), _i64x4(out.stride()), ctypes.c_int64(0), ctypes.c_int64(0), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_prep_rmsnorm_rope_bf16", rc)
    return out


# ---------------------------------------------------------------- element-wise primitives on score tiles
# (the reference's symbols of src/cuda/ffi.rs:349-422; 0 = launched, 1 = not)
def _tile_rc(fn: str, rc: int) -> None:
    if rc != 0:
        raise FlameAttnError(fn, rc)


def tile_causal_mask(scores, q_offset=0, k_offset=0):
    B, H, Q, K = scores.shape
    assert scores.dtype == torch.float32 and scores.is_contiguous()
    _tile_rc("flame_apply_causal_mask_fp32",
             lib().flame_apply_causal_mask_fp32(_ptr(scores), B, H, Q, K, int(q_offset), int(k_offset), _stream()))
    return scores


def tile_attn_mask(scores, mask):
    B, H, Q, K = scores.shape
    assert scores.dtype == torch.float32 and mask.dtype == torch.uint8 and mask.shape == scores.shape
    assert scores.is_contiguous() and mask.is_contiguous()
    _tile_rc("flame_apply_attn_mask_fp32", lib().flame_apply_attn_mask_fp32(_ptr(scores), _ptr(mask), B, H, Q, K, _stream()))
    return scores


def tile_add_mask(logits, user_bool=None, user_add=None, q_abs_start=0, k_abs_start=0, bool_rank=0, add_rank=0, k_total=0,
                  zero_is_mask=True, causal=False):
    BH, q_t, k_t = logits.shape
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    assert user_bool is None or (user_bool.dtype == torch.uint8 and user_bool.is_contiguous())
    assert user_add is None or (user_add.dtype == torch.float32 and user_add.is_contiguous())
    _tile_rc("flame_sdpa_add_mask_tile_fp32",
             lib().flame_sdpa_add_mask_tile_fp32(_ptr(logits), _ptr(user_bool), _ptr(user_add), BH, q_t, k_t, int(q_abs_start),
                                                 int(k_abs_start), int(bool_rank), int(add_rank), int(k_total),
                                                 int(bool(zero_is_mask)), int(bool(causal)), _stream()))
    return logits


def tile_softmax_from_lse(logits, lse_row, out=None):
    BH, q_t, k_t = logits.shape
    assert logits.dtype == torch.float32 and lse_row.dtype == torch.float32 and tuple(lse_row.shape) == (BH, q_t)
    assert logits.is_contiguous() and lse_row.is_contiguous()
    if out is None:
        out = torch.empty(logits.shape, dtype=torch.bfloat16, device=logits.device)
    _tile_rc("flame_sdpa_softmax_from_lse_tile",
             lib().flame_sdpa_softmax_from_lse_tile(_ptr(logits), _ptr(lse_row), _ptr(out), BH, q_t, k_t, _stream()))
    return out


def tile_lse_from_logits(logits):
    BH, q_t, k_t = logits.shape
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    out = torch.empty((BH, q_t), dtype=torch.float32, device=logits.device)
    _tile_rc("flame_sdpa_lse_from_logits_tile",
             lib().flame_sdpa_lse_from_logits_tile(_ptr(logits), _ptr(out), BH, q_t, k_t, _stream()))
    return out


def tile_lse_merge(lse_row, tile_lse_row):
    BH, q_t = lse_row.shape
    assert lse_row.dtype == torch.float32 and tile_lse_row.dtype == torch.float32 and lse_row.shape == tile_lse_row.shape
    assert lse_row.is_contiguous() and tile_lse_row.is_contiguous()
    _tile_rc("flame_sdpa_lse_merge_rows", lib().flame_sdpa_lse_merge_rows(_ptr(lse_row), _ptr(tile_lse_row), BH, q_t, _stream()))
    return lse_row


def tile_dropout(probs, p, seed):
    BH, q_t, k_t = probs.shape
    assert probs.dtype == torch.bfloat16 and probs.is_contiguous()
    _tile_rc("flame_sdpa_dropout_bf16_inplace",
             lib().flame_sdpa_dropout_bf16_inplace(_ptr(probs), ctypes.c_float(p), ctypes.c_uint64(seed & (2 ** 64 - 1)),
                                                   BH, q_t, k_t, _stream()))
    return probs


# ---------------------------------------------------------------- FP8 form of offloaded activations
def bf16_to_fp8(x, inv_scale, out=None):
    """out[i] = fp8_e4m3(float(x[i]) * inv_scale) (uint8), flame_bf16_to_fp8; x is any contiguous bf16 tensor."""
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device) if out is None else out
    assert out.dtype == torch.uint8 and out.is_contiguous() and out.numel() == x.numel()
    rc = lib().flame_bf16_to_fp8(_ptr(x), _ptr(out), ctypes.c_float(inv_scale), ctypes.c_size_t(x.numel()), _stream())
    if rc != 0:
        raise FlameAttnError("flame_bf16_to_fp8", rc)
    return out


def fp8_to_bf16(codes, scale, out=None):
    """out[i] = bf16(float(fp8(codes[i])) * scale), flame_fp8_to_bf16."""
    assert codes.dtype == torch.uint8 and codes.is_contiguous()
    out = torch.empty(codes.shape, dtype=torch.bfloat16, device=codes.device) if out is None else out
    assert out.dtype == torch.bfloat16 and out.is_contiguous() and out.numel() == codes.numel()
    rc = lib().flame_fp8_to_bf16(_ptr(codes), _ptr(out), ctypes.c_float(scale), ctypes.c_size_t(codes.numel()), _stream())
    if rc != 0:
        raise FlameAttnError("flame_fp8_to_bf16", rc)
    return out


# ---------------------------------------------------------------- dropout of the probabilities
def attn_fwd_dropout(q, k, v, scale, dropout_p, dropout_seed, causal=False, kv_len=None, mask=None, out=None,
                     draw_chunk_q=0, draw_chunk_kv=0):
    """O, LSE = flame_attn_fwd_dropout_tiled_bf16(...): the kept set of the reference's autograd_v4 operator for this
    seed; draw_chunk_q / draw_chunk_kv: the tiles it draws over when it is chunked (0 = the whole axis)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    o = torch.empty((B, H, Sq, D), dtype=torch.bfloat16, device=q.device) if out is None else out
    lse = torch.empty((B * H, Sq), dtype=torch.float32, device=q.device)
    rc = lib().flame_attn_fwd_dropout_tiled_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, H, Sq, Sk, D, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        *(ctypes.c_int64(0) for _ in range(5)),
        int(bool(causal)), _ptr(kv_len), _ptr(mask), _mask_strides(mask, B, H, Sq, Sk),
        ctypes.c_float(dropout_p), ctypes.c_uint64(dropout_seed & (2 ** 64 - 1)), int(draw_chunk_q), int(draw_chunk_kv), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_fwd_dropout_tiled_bf16", rc)
    return o, lse


def attn_bwd_dropout(q, k, v, o, do, lse, scale, dropout_p, dropout_seed, causal=False, kv_len=None, mask=None, workspace=None,
                     draw_chunk_q=0, draw_chunk_kv=0):
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    if workspace is None:
        workspace = torch.empty(bwd_workspace_bytes(B, H, Sq, D), dtype=torch.uint8, device=q.device)
    dq = torch.empty((B, H, Sq, D), dtype=torch.bfloat16, device=q.device)
    dk = torch.empty((B, H, Sk, D), dtype=torch.bfloat16, device=q.device)
    dv = torch.empty((B, H, Sk, D), dtype=torch.bfloat16, device=q.device)
    rc = lib().flame_attn_bwd_dropout_tiled_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
        B, H, Sq, Sk, D, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        _i64x4(do.stride()), _i64x4(dq.stride()), _i64x4(dk.stride()), _i64x4(dv.stride()),
        *(ctypes.c_int64(0) for _ in range(9)),
        int(bool(causal)), _ptr(kv_len), _ptr(mask), _mask_strides(mask, B, H, Sq, Sk),
        ctypes.c_float(dropout_p), ctypes.c_uint64(dropout_seed & (2 ** 64 - 1)), int(draw_chunk_q), int(draw_chunk_kv),
        _ptr(workspace), ctypes.c_size_t(workspace.numel()), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_bwd_dropout_tiled_bf16", rc)
    return dq, dk, dv


def materialised_workspace_bytes(B, H, Sq, Sk, D, Dv, backward) -> int:
    f = lib().flame_attn_materialised_workspace_bytes
    f.restype = ctypes.c_size_t
    return int(f(B, H, Sq, Sk, D, Dv, int(bool(backward))))


def _bias_strides(bias, B, H, Sq, Sk):
    if bias is None:
        return None
    full = (B, H, Sq, Sk)
    st = []
    for ax in range(4):
        assert bias.shape[ax] in (1, full[ax]), "bias is not broadcastable to [B,H,Sq,Sk]"
        st.append(0 if (bias.shape[ax] == 1 and full[ax] != 1) else bias.stride(ax))
    return _i64x4(st)


def attn_fwd_materialised(q, k, v, scale, causal=False, kv_len=None, mask=None, bias=None, want_lse=True, out=None, workspace=None,
                          dropout_p=0.0, dropout_seed=0, draw_chunk_q=0, draw_chunk_kv=0):
    """O, LSE = flame_attn_fwd_materialised_bf16(...): any head dim, a value head dim of its own, mask, bias, dropout."""
    B, H, Sq, D = q.shape
    Sk, Dv = k.shape[2], v.shape[3]
    o = torch.empty((B, H, Sq, Dv), dtype=torch.bfloat16, device=q.device) if out is None else out
    lse = torch.empty((B * H, Sq), dtype=torch.float32, device=q.device) if want_lse else None
    if workspace is None:
        workspace = torch.empty(materialised_workspace_bytes(B, H, Sq, Sk, D, Dv, False), dtype=torch.uint8, device=q.device)
    rc = lib().flame_attn_fwd_materialised_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, H, Sq, Sk, D, Dv, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        *(ctypes.c_int64(0) for _ in range(5)),
        int(bool(causal)), _ptr(kv_len), _ptr(mask), _mask_strides(mask, B, H, Sq, Sk),
        _ptr(bias), 1 if (bias is not None and bias.dtype == torch.float32) else 0, _bias_strides(bias, B, H, Sq, Sk),
        ctypes.c_float(dropout_p), ctypes.c_uint64(dropout_seed & (2 ** 64 - 1)), int(draw_chunk_q), int(draw_chunk_kv),
        _ptr(workspace), ctypes.c_size_t(workspace.numel()), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_fwd_materialised_bf16", rc)
    return o, lse


def attn_bwd_materialised(q, k, v, o, do, lse, scale, causal=False, kv_len=None, mask=None, workspace=None, grads=None,
                          dropout_p=0.0, dropout_seed=0, draw_chunk_q=0, draw_chunk_kv=0):
    """dQ, dK, dV = flame_attn_bwd_materialised_bf16(...)."""
    B, H, Sq, D = q.shape
    Sk, Dv = k.shape[2], v.shape[3]
    if workspace is None:
        workspace = torch.empty(materialised_workspace_bytes(B, H, Sq, Sk, D, Dv, True), dtype=torch.uint8, device=q.device)
    if grads is None:
        grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    dq, dk, dv = grads
    rc = lib().flame_attn_bwd_materialised_bf16(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
        B, H, Sq, Sk, D, Dv, ctypes.c_float(scale),
        _i64x4(q.stride()), _i64x4(k.stride()), _i64x4(v.stride()), _i64x4(o.stride()),
        _i64x4(do.stride()), _i64x4(dq.stride()), _i64x4(dk.stride()), _i64x4(dv.stride()),
        *(ctypes.c_int64(0) for _ in range(9)),
        int(bool(causal)), _ptr(kv_len), _ptr(mask), _mask_strides(mask, B, H, Sq, Sk),
        ctypes.c_float(dropout_p), ctypes.c_uint64(dropout_seed & (2 ** 64 - 1)), int(draw_chunk_q), int(draw_chunk_kv),
        _ptr(workspace), ctypes.c_size_t(workspace.numel()), _stream())
    if rc != 0:
        raise FlameAttnError("flame_attn_bwd_materialised_bf16", rc)
    return dq, dk, dv
