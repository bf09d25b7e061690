"""ctypes front end of the CPU oracle (``sdpa_oracle.c``) plus tiny fp64 brute-force twins.

TEST INFRASTRUCTURE ONLY: importable from ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; never from the product package.

bf16 tensors are numpy ``uint16`` arrays holding the raw bit patterns, contiguous ``[B,H,S,D]``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``sdpa_oracle.c`` with gcc (``make -C oracle``)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def set_num_threads(n: int) -> None:
    lib().oracle_set_num_threads(ctypes.c_int(n))


# ---------------------------------------------------------------- bf16 helpers (numpy)
def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------- C oracle wrappers
def _mask_args(mask, B, H, Sq, Sk):
    """mask: uint8 array broadcastable to [B,H,Sq,Sk] (4-D, dims of size 1 broadcast)."""
    if mask is None:
        return None, (0, 0, 0, 0), None
    m = np.ascontiguousarray(mask, dtype=np.uint8)
    assert m.ndim == 4, "mask must be 4-D"
    full = (B, H, Sq, Sk)
    st = []
    for ax in range(4):
        assert m.shape[ax] in (1, full[ax]), f"mask dim {ax} not broadcastable"
        st.append(0 if m.shape[ax] == 1 and full[ax] != 1 else m.strides[ax])
    return m, tuple(st), m


def sdpa_fwd(q, k, v, scale, causal=False, kv_len=None, mask=None, heads=None, want_f32=False, rows=None):
    """Naive fp32 forward. Returns (O bf16-bits, LSE fp32[, O fp32]).

    heads = (begin, end) over the flat b*H+h index and rows = (begin, end) over the query rows restrict
    the work; the outputs keep their full shapes and only that part of them is filled."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    q, k, v = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k, v))
    O = np.zeros((B, H, Sq, D), np.uint16)
    LSE = np.zeros((B, H, Sq), np.float32)
    O32 = np.zeros((B, H, Sq, D), np.float32) if want_f32 else None
    kvl = None if kv_len is None else np.ascontiguousarray(kv_len, dtype=np.int32)
    m, st, _keep = _mask_args(mask, B, H, Sq, Sk)
    hb, he = (0, B * H) if heads is None else heads
    rb, re_ = (0, Sq) if rows is None else rows
    rc = lib().oracle_sdpa_fwd_rows(
        _p(q), _p(k), _p(v), B, H, Sq, Sk, D, ctypes.c_float(scale), int(bool(causal)),
        _p(kvl), _p(m), *(ctypes.c_int64(s) for s in st), hb, he, rb, re_, _p(O), _p(LSE), _p(O32))
    if rc != 0:
        raise RuntimeError(f"oracle_sdpa_fwd failed: {rc}")
    return (O, LSE, O32) if want_f32 else (O, LSE)


def sdpa_fwd_bias(q, k, v, scale, bias, want_f32=False):
    """Naive fp32 forward with an additive fp32 bias [B|1, H|1, Sq, Sk] on the scaled logits."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    q, k, v = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k, v))
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    assert bias.ndim == 4 and bias.shape[2:] == (Sq, Sk) and bias.shape[0] in (1, B) and bias.shape[1] in (1, H)
    st = [0 if bias.shape[i] == 1 and i < 2 else bias.strides[i] // 4 for i in range(4)]
    O = np.zeros((B, H, Sq, D), np.uint16)
    LSE = np.zeros((B, H, Sq), np.float32)
    O32 = np.zeros((B, H, Sq, D), np.float32) if want_f32 else None
    rc = lib().oracle_sdpa_fwd_bias(
        _p(q), _p(k), _p(v), B, H, Sq, Sk, D, ctypes.c_float(scale), _p(bias),
        *(ctypes.c_int64(s_) for s_ in st), _p(O), _p(LSE), _p(O32))
    if rc != 0:
        raise RuntimeError(f"oracle_sdpa_fwd_bias failed: {rc}")
    return (O, LSE, O32) if want_f32 else (O, LSE)


def sdpa_bwd(q, k, v, o, do, scale, causal=False, kv_len=None, mask=None, heads=None, want_f32=False, rows=None):
    """Naive fp32 backward. Returns (dQ, dK, dV) bf16 bits [+ fp32 copies].

    With rows = (begin, end) only those query rows take part: dQ is filled for them, and dK / dV are
    the sums over them (complete for every key that no query outside the band attends to)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    q, k, v, o, do = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k, v, o, do))
    dQ = np.zeros((B, H, Sq, D), np.uint16)
    dK = np.zeros((B, H, Sk, D), np.uint16)
    dV = np.zeros((B, H, Sk, D), np.uint16)
    f = [np.zeros(t.shape, np.float32) for t in (dQ, dK, dV)] if want_f32 else [None] * 3
    kvl = None if kv_len is None else np.ascontiguousarray(kv_len, dtype=np.int32)
    m, st, _keep = _mask_args(mask, B, H, Sq, Sk)
    hb, he = (0, B * H) if heads is None else heads
    rb, re_ = (0, Sq) if rows is None else rows
    rc = lib().oracle_sdpa_bwd_rows(
        _p(q), _p(k), _p(v), _p(o), _p(do), B, H, Sq, Sk, D, ctypes.c_float(scale),
        int(bool(causal)), _p(kvl), _p(m), *(ctypes.c_int64(s) for s in st), hb, he, rb, re_,
        _p(dQ), _p(dK), _p(dV), _p(f[0]), _p(f[1]), _p(f[2]))
    if rc != 0:
        raise RuntimeError(f"oracle_sdpa_bwd failed: {rc}")
    return (dQ, dK, dV, *f) if want_f32 else (dQ, dK, dV)


def sage_quant(q, k, qblk=128, kblk=64, smooth_k=True):
    """Returns dict(kmean, ks, qi8, ki8, sq, sk)."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    q, k = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k))
    nqb, nkb = -(-Sq // qblk), -(-Sk // kblk)
    out = dict(
        kmean=np.zeros((B, H, D), np.float32), ks=np.zeros((B, H, Sk, D), np.uint16),
        qi8=np.zeros((B, H, Sq, D), np.int8), ki8=np.zeros((B, H, Sk, D), np.int8),
        sq=np.zeros((B, H, nqb), np.float32), sk=np.zeros((B, H, nkb), np.float32))
    rc = lib().oracle_sage_quant(
        _p(q), _p(k), B, H, Sq, Sk, D, qblk, kblk, int(bool(smooth_k)),
        _p(out["kmean"]), _p(out["ks"]), _p(out["qi8"]), _p(out["ki8"]), _p(out["sq"]), _p(out["sk"]))
    if rc != 0:
        raise RuntimeError(f"oracle_sage_quant failed: {rc}")
    return out


def sage_fwd(qi8, ki8, sq, sk, v, scale, qblk=128, kblk=64, causal=False, heads=None, kv_len=None, rows=None,
             want_f32=False, bias=None):
    """Sage forward from quantised operands. Returns (O bf16 bits, LSE[, O fp32])."""
    B, H, Sq, D = qi8.shape
    Sk = ki8.shape[2]
    qi8, ki8 = (np.ascontiguousarray(t, dtype=np.int8) for t in (qi8, ki8))
    sq, sk = (np.ascontiguousarray(t, dtype=np.float32) for t in (sq, sk))
    v = np.ascontiguousarray(v, dtype=np.uint16)
    O = np.zeros((B, H, Sq, D), np.uint16)
    LSE = np.zeros((B, H, Sq), np.float32)
    O32 = np.zeros((B, H, Sq, D), np.float32) if want_f32 else None
    kvl = None if kv_len is None else np.ascontiguousarray(kv_len, dtype=np.int32)
    hb, he = (0, B * H) if heads is None else heads
    rb, re_ = (0, Sq) if rows is None else rows
    bst = (0, 0, 0, 0)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
        assert bias.ndim == 4 and bias.shape[2:] == (Sq, Sk) and bias.shape[0] in (1, B) and bias.shape[1] in (1, H)
        bst = tuple(0 if bias.shape[i] == 1 and i < 2 else bias.strides[i] // 4 for i in range(4))
    rc = lib().oracle_sage_fwd(_p(qi8), _p(ki8), _p(sq), _p(sk), _p(v), B, H, Sq, Sk, D, qblk, kblk,
                               ctypes.c_float(scale), int(bool(causal)), _p(kvl),
                               _p(bias), *(ctypes.c_int64(x) for x in bst), hb, he, rb, re_,
                               _p(O), _p(LSE), _p(O32))
    if rc != 0:
        raise RuntimeError(f"oracle_sage_fwd failed: {rc}")
    return (O, LSE, O32) if want_f32 else (O, LSE)


# ---------------------------------------------------------------- fp64 brute force (checker of the checker)
def brute_sdpa_f64(q, k, v, scale, keep=None, bias=None):
    """Pure numpy fp64 attention on float arrays [.., Sq, D]; keep: bool [.., Sq, Sk] or None; bias: additive,
    broadcastable to [.., Sq, Sk], or None.

    Returns (O, LSE, P), all fp64.  Written from the textbook definition, not from the C file.
    """
    q, k, v = (np.asarray(t, np.float64) for t in (q, k, v))
    s = np.einsum("...id,...jd->...ij", q, k) * float(scale)
    if bias is not None:
        s = s + np.asarray(bias, np.float64)
    if keep is not None:
        s = np.where(keep, s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    msafe = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - msafe)
    l = e.sum(axis=-1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        p = np.where(l > 0, e / np.where(l > 0, l, 1.0), 0.0)
        lse = np.where(l[..., 0] > 0, msafe[..., 0] + np.log(np.where(l[..., 0] > 0, l[..., 0], 1.0)), -np.inf)
    return p @ v, lse, p


# ---------------------------------------------------------------- error metrics used by every parity test
def max_abs(a, b) -> float:
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)))) if np.size(a) else 0.0


def rel_l2(a, b) -> float:
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    den = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / den) if den > 0 else float(np.linalg.norm(a - b))


def cosine(a, b) -> float:
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    den = np.linalg.norm(a) * np.linalg.norm(b)
    return float(a @ b / den) if den > 0 else 1.0


def prep_rmsnorm_rope(x_bnhd, weight=None, cos=None, sin=None, eps=1e-6, apply_norm=True):
    """Input preparation of joint attention, restated from the reference's two kernels run back to back.

    x_bnhd: uint16 bf16 bits [B,N,H,D]; weight: bf16 bits [D] or None; cos/sin: fp32 [N,D/2] (pass
    bf16 tables already widened to fp32).  Returns bf16 bits [B,H,N,D].

      fused_rms_norm.cu:26-86   v = bf16(x * rsqrt(mean(x^2) + eps) * w), fp32 arithmetic
      bf16_ops.rs:361-394       y[2p] = bf16(v[2p] c - v[2p+1] s), y[2p+1] = bf16(v[2p] s + v[2p+1] c)

    Plain IEEE fp32 without contraction; the mean of squares is accumulated in fp64 and rounded once
    (the reference's summation order is a property of its launch shape, not of the algorithm).
    Pinned by the reference's RoPE known-answer test and by closed forms (see tests)."""
    x = bf16_to_f32(np.asarray(x_bnhd))
    if apply_norm:
        ms = np.mean(x.astype(np.float64) ** 2, axis=-1, keepdims=True).astype(np.float32)
        with np.errstate(divide="ignore", invalid="ignore"):       # eps = 0 on an all-zero row
            rs = (np.float32(1.0) / np.sqrt(ms + np.float32(eps), dtype=np.float32)).astype(np.float32)
            v = (x * rs).astype(np.float32)
        if weight is not None:
            v = (v * bf16_to_f32(np.asarray(weight))).astype(np.float32)
        x = bf16_to_f32(f32_to_bf16(v))
    x = np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3)))          # [B,H,N,D]
    if cos is not None:
        c = np.asarray(cos, np.float32)[None, None]
        s_ = np.asarray(sin, np.float32)[None, None]
        e, o = x[..., 0::2], x[..., 1::2]
        y = np.empty_like(x)
        y[..., 0::2] = (e * c).astype(np.float32) - (o * s_).astype(np.float32)
        y[..., 1::2] = (e * s_).astype(np.float32) + (o * c).astype(np.float32)
        x = y
    return f32_to_bf16(x)


# ---------------------------------------------------------------- element-wise primitives on score tiles
# (tile_ops_oracle.c; reference: src/kernels/sdpa_kernels.cu).  Arrays are modified in place where the
# reference's kernels work in place; the result is returned as well.
def tile_causal_mask(scores: np.ndarray, q_offset: int, k_offset: int) -> np.ndarray:
    B, H, Q, K = scores.shape
    assert scores.dtype == np.float32 and scores.flags.c_contiguous
    lib().oracle_tile_causal_mask(_p(scores), B, H, Q, K, int(q_offset), int(k_offset))
    return scores


def tile_attn_mask(scores: np.ndarray, mask: np.ndarray) -> np.ndarray:
    assert scores.dtype == np.float32 and mask.dtype == np.uint8 and scores.shape == mask.shape
    assert scores.flags.c_contiguous and mask.flags.c_contiguous
    lib().oracle_tile_attn_mask(_p(scores), _p(mask), ctypes.c_int64(scores.size))
    return scores


def tile_add_mask(logits: np.ndarray, user_bool=None, user_add=None, q_abs_start=0, k_abs_start=0, bool_rank=0,
                  add_rank=0, k_total=0, zero_is_mask=True, causal=False) -> np.ndarray:
    BH, q_t, k_t = logits.shape
    assert logits.dtype == np.float32 and logits.flags.c_contiguous
    if user_bool is not None:
        assert user_bool.dtype == np.uint8 and user_bool.flags.c_contiguous
    if user_add is not None:
        assert user_add.dtype == np.float32 and user_add.flags.c_contiguous
    lib().oracle_tile_add_mask(_p(logits), _p(user_bool), _p(user_add), BH, q_t, k_t, int(q_abs_start), int(k_abs_start),
                               int(bool_rank), int(add_rank), int(k_total), int(bool(zero_is_mask)), int(bool(causal)))
    return logits


def tile_softmax_from_lse(logits: np.ndarray, lse_row: np.ndarray):
    """Returns (bf16 bit patterns, the fp32 values before rounding)."""
    BH, q_t, k_t = logits.shape
    assert logits.dtype == np.float32 and lse_row.dtype == np.float32 and lse_row.shape == (BH, q_t)
    probs = np.empty(logits.shape, np.uint16)
    p32 = np.empty(logits.shape, np.float32)
    lib().oracle_tile_softmax_from_lse(_p(np.ascontiguousarray(logits)), _p(np.ascontiguousarray(lse_row)), _p(probs), _p(p32),
                                       BH, q_t, k_t)
    return probs, p32


def tile_lse_from_logits(logits: np.ndarray) -> np.ndarray:
    BH, q_t, k_t = logits.shape
    assert logits.dtype == np.float32
    out = np.empty((BH, q_t), np.float32)
    lib().oracle_tile_lse_from_logits(_p(np.ascontiguousarray(logits)), _p(out), BH, q_t, k_t)
    return out


def tile_lse_merge(lse_row: np.ndarray, tile_lse_row: np.ndarray) -> np.ndarray:
    assert lse_row.dtype == np.float32 and tile_lse_row.dtype == np.float32 and lse_row.shape == tile_lse_row.shape
    assert lse_row.flags.c_contiguous and tile_lse_row.flags.c_contiguous
    lib().oracle_tile_lse_merge(_p(lse_row), _p(tile_lse_row), ctypes.c_int64(lse_row.size))
    return lse_row


def tile_uniform01(seed: int, b: int, qi: int, kj: int) -> float:
    f = lib().oracle_tile_uniform01
    f.restype = ctypes.c_float
    return float(f(ctypes.c_uint64(seed & (2 ** 64 - 1)), int(b), int(qi), int(kj)))


def tile_dropout(probs: np.ndarray, p: float, seed: int) -> np.ndarray:
    BH, q_t, k_t = probs.shape
    assert probs.dtype == np.uint16 and probs.flags.c_contiguous
    lib().oracle_tile_dropout(_p(probs), ctypes.c_float(p), ctypes.c_uint64(seed & (2 ** 64 - 1)), BH, q_t, k_t)
    return probs


# ---------------------------------------------------------------- dropout of the probabilities
# (the reference's autograd_v4 operator, unchunked: src/autograd_v4/ops/sdpa.rs:229-231, :600-649; src/rng/mod.rs:14-24)
def dropout_keep(seed: int, flat_index: int, p: float) -> bool:
    return bool(lib().oracle_dropout_keep(ctypes.c_uint64(seed & (2 ** 64 - 1)), ctypes.c_uint64(flat_index), ctypes.c_float(p)))


def dropout_keep_tiled(seed: int, bh: int, i: int, j: int, Sq: int, Sk: int, cq: int, ck: int, p: float) -> bool:
    return bool(lib().oracle_dropout_keep_tiled(ctypes.c_uint64(seed & (2 ** 64 - 1)), bh, i, j, Sq, Sk, cq, ck, ctypes.c_float(p)))


def _xorshift_uniform(seed32: np.ndarray, idx32: np.ndarray) -> np.ndarray:
    s = idx32.astype(np.uint32) ^ seed32.astype(np.uint32)
    s ^= s << np.uint32(13)
    s ^= s >> np.uint32(17)
    s ^= s << np.uint32(5)
    return (s >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)


def dropout_uniforms(B, H, Sq, Sk, seed, chunk_q=0, chunk_kv=0) -> np.ndarray:
    """fp32 [B,H,Sq,Sk]: the uniform each probability is compared with, written from the recurrence in numpy (not
    through the C file).  chunk_q / chunk_kv: the tiles of a chunked draw (0 = the whole axis)."""
    cq = Sq if chunk_q <= 0 or chunk_q > Sq else chunk_q
    ck = Sk if chunk_kv <= 0 or chunk_kv > Sk else chunk_kv
    bh = np.arange(B * H, dtype=np.uint64)[:, None, None]
    i = np.arange(Sq, dtype=np.uint64)[None, :, None]
    j = np.arange(Sk, dtype=np.uint64)[None, None, :]
    q_off, k_off = (i // cq) * cq, (j // ck) * ck
    q_t, k_t = np.minimum(cq, Sq - q_off), np.minimum(ck, Sk - k_off)
    idx = (bh * q_t + (i - q_off)) * k_t + (j - k_off)
    seed32 = (np.uint64(seed & 0xFFFFFFFF) + k_off) & np.uint64(0xFFFFFFFF)          # the query offset sits above bit 31
    u = _xorshift_uniform(np.broadcast_to(seed32, idx.shape), idx & np.uint64(0xFFFFFFFF))
    return u.reshape(B, H, Sq, Sk)


def dropout_keep_mask(B, H, Sq, Sk, p, seed, chunk_q=0, chunk_kv=0) -> np.ndarray:
    """bool [B,H,Sq,Sk]: kept where the uniform is >= p."""
    return dropout_uniforms(B, H, Sq, Sk, seed, chunk_q, chunk_kv) >= np.float32(p)


class operand_rounding:
    """Context manager: inside it the oracle rounds the left operands of P V, P^T dO, dS K and dS^T Q to bf16, as a
    kernel that forms those products on a bf16 matrix unit must (oracle_set_operand_rounding in sdpa_oracle.c)."""

    def __enter__(self):
        lib().oracle_set_operand_rounding(1)
        return self

    def __exit__(self, *exc):
        lib().oracle_set_operand_rounding(0)
        return False


def sdpa_fwd_dropout(q, k, v, scale, p, seed, causal=False, kv_len=None, mask=None, want_f32=False, chunk_q=0, chunk_kv=0):
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    q, k, v = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k, v))
    O = np.zeros((B, H, Sq, D), np.uint16)
    LSE = np.zeros((B, H, Sq), np.float32)
    O32 = np.zeros((B, H, Sq, D), np.float32) if want_f32 else None
    kvl = None if kv_len is None else np.ascontiguousarray(kv_len, dtype=np.int32)
    m, st, _keep = _mask_args(mask, B, H, Sq, Sk)
    rc = lib().oracle_sdpa_fwd_dropout(_p(q), _p(k), _p(v), B, H, Sq, Sk, D, ctypes.c_float(scale), int(bool(causal)), _p(kvl),
                                       _p(m), *(ctypes.c_int64(x) for x in st), ctypes.c_float(p), ctypes.c_uint64(seed & (2 ** 64 - 1)), int(chunk_q), int(chunk_kv),
                                       _p(O), _p(LSE), _p(O32))
    if rc != 0:
        raise RuntimeError(f"oracle_sdpa_fwd_dropout failed: {rc}")
    return (O, LSE, O32) if want_f32 else (O, LSE)


def sdpa_bwd_dropout(q, k, v, o, do, scale, p, seed, causal=False, kv_len=None, mask=None, want_f32=False, chunk_q=0, chunk_kv=0):
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    q, k, v, o, do = (np.ascontiguousarray(t, dtype=np.uint16) for t in (q, k, v, o, do))
    dQ = np.zeros((B, H, Sq, D), np.uint16)
    dK = np.zeros((B, H, Sk, D), np.uint16)
    dV = np.zeros((B, H, Sk, D), np.uint16)
    f = [np.zeros(t.shape, np.float32) for t in (dQ, dK, dV)] if want_f32 else [None] * 3
    kvl = None if kv_len is None else np.ascontiguousarray(kv_len, dtype=np.int32)
    m, st, _keep = _mask_args(mask, B, H, Sq, Sk)
    rc = lib().oracle_sdpa_bwd_dropout(_p(q), _p(k), _p(v), _p(o), _p(do), B, H, Sq, Sk, D, ctypes.c_float(scale),
                                       int(bool(causal)), _p(kvl), _p(m), *(ctypes.c_int64(x) for x in st), ctypes.c_float(p), ctypes.c_uint64(seed & (2 ** 64 - 1)),
                                       int(chunk_q), int(chunk_kv), _p(dQ), _p(dK), _p(dV), _p(f[0]), _p(f[1]), _p(f[2]))
    if rc != 0:
        raise RuntimeError(f"oracle_sdpa_bwd_dropout failed: {rc}")
    return (dQ, dK, dV, *f) if want_f32 else (dQ, dK, dV)


# --------------------------------------------------------------------------- FP8 form of offloaded activations
def f32_to_fp8_e4m3(val: float) -> int:
    """The reference's scalar encoder (src/cuda/fp8_quant.cu:19-57) on one fp32 product."""
    f = lib().oracle_f32_to_fp8_e4m3
    f.restype = ctypes.c_uint8
    return int(f(ctypes.c_float(val)))


def bf16_to_fp8(x_bits: np.ndarray, inv_scale: float) -> np.ndarray:
    """out[i] = fp8(bf16(x[i]) * inv_scale), src/cuda/fp8_quant.cu:59-72."""
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    out = np.empty(x.shape, np.uint8)
    lib().oracle_bf16_to_fp8(_p(x), _p(out), ctypes.c_float(inv_scale), ctypes.c_size_t(x.size))
    return out


def fp8_to_bf16(codes: np.ndarray, scale: float) -> np.ndarray:
    """out[i] = bf16(fp8(codes[i]) * scale), src/cuda/fp8_dequant.cu:10-39."""
    c = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(c.shape, np.uint16)
    lib().oracle_fp8_to_bf16(_p(c), _p(out), ctypes.c_float(scale), ctypes.c_size_t(c.size))
    return out
