"""Seeded synthetic inputs for the five benchmark / parity configurations of the attention path.

Counter-based generator (SplitMix64 hash of ``(seed, stream, index)`` -> Box-Muller) so any slice
of any tensor can be regenerated independently and identically on every machine.  All values are
rounded to bf16 (round-to-nearest-even) and returned as raw ``uint16`` bit patterns, contiguous
``[B,H,S,D]``; both the CPU checker and the HIP kernels consume exactly these bits.

The input preparation of the joint text+image configuration follows the reference's conventions:
per-row RMS normalisation ``x * rsqrt(mean(x^2) + 1e-6)`` (scripts/generate_klein_joint_attn_fixture.py:49-52),
interleaved-pair rotary embedding ``(x0 cos - x1 sin, x0 sin + x1 cos)`` on pairs ``(2p, 2p+1)``
(src/bf16_ops.rs:384-390, src/tests/attention_tests.rs:8-34), text tokens first
(scripts/generate_klein_joint_attn_fixture.py:113-116).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

SEED_BASE = 0xF1A4E000
_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def normal_f32(seed: int, stream: int, n: int, chunk: int = 1 << 22) -> np.ndarray:
    """n i.i.d. N(0,1) samples as fp32, a pure function of (seed, stream, index)."""
    key = _splitmix64(np.array([(seed * 0x100000001B3 + stream) & 0xFFFFFFFFFFFFFFFF], np.uint64))[0]
    out = np.empty(n, np.float32)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        idx = np.arange(lo, hi, dtype=np.uint64)
        with np.errstate(over="ignore"):
            a = _splitmix64(key + np.uint64(2) * idx)
            b = _splitmix64(key + np.uint64(2) * idx + np.uint64(1))
        u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
        u2 = (b >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        out[lo:hi] = (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * math.pi * u2)).astype(np.float32)
    return out


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    return r.astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


@dataclass
class Workload:
    name: str
    q: np.ndarray
    k: np.ndarray
    v: np.ndarray
    do: Optional[np.ndarray]
    scale: float
    causal: bool = False
    kv_len: Optional[np.ndarray] = None          # int32 [B]
    mask: Optional[np.ndarray] = None            # uint8 keep-mask, 4-D broadcastable
    note: str = ""
    extra: dict = field(default_factory=dict)

    @property
    def shape(self):
        B, H, Sq, D = self.q.shape
        return B, H, Sq, self.k.shape[2], D

    def valid_pairs(self) -> int:
        """Number of (query, key) pairs that are attended, summed over batch and heads."""
        B, H, Sq, Sk, _ = self.shape
        if self.kv_len is not None:
            lens = [int(x) for x in self.kv_len]
        else:
            lens = [Sk] * B
        total = 0
        for L in lens:
            if self.causal:
                # key j attends to query i when j <= i and j < L
                n = min(L, Sq)
                total += n * (n + 1) // 2 + (Sq - n) * L
            else:
                total += Sq * L
        return total * H

    def flops(self, fwd: bool = True, bwd: bool = True) -> float:
        """Algorithmic FLOPs: forward two GEMMs (4*pairs*D), backward five GEMMs (10*pairs*D)."""
        D = self.shape[4]
        per_pair = (4 if fwd else 0) + (10 if bwd else 0)
        return float(per_pair) * self.valid_pairs() * D

    def saved_activation_bytes(self) -> dict:
        """What this path keeps between forward and backward, next to a materialised softmax."""
        B, H, Sq, Sk, D = self.shape
        return {
            "O_bf16": B * H * Sq * D * 2,
            "LSE_f32": B * H * Sq * 4,
            "materialised_P_bf16": B * H * Sq * Sk * 2,
            "materialised_P_f32": B * H * Sq * Sk * 4,
        }


def _gauss(seed, stream, shape, mul=1.0):
    x = normal_f32(seed, stream, int(np.prod(shape))).reshape(shape)
    if mul != 1.0:
        x = x * np.float32(mul)
    return x


def config1(B=1, H=4, S=256, D=64) -> Workload:
    """Small non-causal SDPA, CPU-runnable."""
    seed = SEED_BASE + 1
    t = [f32_to_bf16_bits(_gauss(seed, s, (B, H, S, D))) for s in range(4)]
    return Workload("cfg1_small_noncausal", t[0], t[1], t[2], t[3], 1.0 / math.sqrt(D))


def rms_normalise(x: np.ndarray, eps: float = 1e-6) -> np.ndarray:
    x = x.astype(np.float32)
    ms = np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32)
    return x * (1.0 / np.sqrt(ms + np.float32(eps))).astype(np.float32)


def axial_rope_tables(n_text: int, grid_h: int, grid_w: int, D: int, theta: float = 10000.0):
    """cos/sin [S, D/2] fp32 for text-first joint sequences.

    Pair p < D/4 rotates by the row position y, pair p >= D/4 by the column position x, with
    frequency theta^(-(p mod D/4)/(D/4)).  Text token t sits at (y,x) = (t,t); image token
    n = n_text + grid_w*r + c sits at (r,c).
    """
    half = D // 2
    quarter = half // 2
    S = n_text + grid_h * grid_w
    y = np.empty(S, np.float32)
    x = np.empty(S, np.float32)
    y[:n_text] = x[:n_text] = np.arange(n_text, dtype=np.float32)
    r, c = np.divmod(np.arange(grid_h * grid_w), grid_w)
    y[n_text:] = r
    x[n_text:] = c
    p = np.arange(half)
    freq = (theta ** (-(p % quarter).astype(np.float64) / quarter)).astype(np.float32)
    pos = np.where((p < quarter)[None, :], y[:, None], x[:, None]).astype(np.float32)
    ang = pos * freq[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def apply_rope_interleaved(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x [..., S, D] fp32; pairs (2p, 2p+1) are rotated by the angle of table row s, column p."""
    x0 = x[..., 0::2]
    x1 = x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = x0 * cos - x1 * sin
    out[..., 1::2] = x0 * sin + x1 * cos
    return out


def config2(B=1, H=24, n_text=512, grid=64, D=128) -> Workload:
    """DiT joint text+image attention at production shape (4608 tokens for the defaults)."""
    seed = SEED_BASE + 2
    S = n_text + grid * grid
    cos, sin = axial_rope_tables(n_text, grid, grid, D)
    qk = []
    for s in range(2):
        x = rms_normalise(_gauss(seed, s, (B, H, S, D)))
        qk.append(f32_to_bf16_bits(apply_rope_interleaved(x, cos, sin)))
    v = f32_to_bf16_bits(_gauss(seed, 2, (B, H, S, D)))
    do = f32_to_bf16_bits(_gauss(seed, 3, (B, H, S, D)))
    return Workload("cfg2_dit_joint_4608" if S == 4608 else f"cfg2_dit_joint_{S}",
                    qk[0], qk[1], v, do, 1.0 / math.sqrt(D),
                    note="Q,K unit-RMS rows + axial interleaved RoPE; V,dO N(0,1)")


def config3(B=4, H=16, Sq=1024, lens=(77, 333, 1024, 2049), D=64, garbage=1.0e4) -> Workload:
    """Ragged key-length cross attention; the padded tail of K and V holds large finite garbage."""
    seed = SEED_BASE + 3
    assert len(lens) == B
    Sk = max(lens)
    q = f32_to_bf16_bits(_gauss(seed, 0, (B, H, Sq, D)))
    k = _gauss(seed, 1, (B, H, Sk, D))
    v = _gauss(seed, 2, (B, H, Sk, D))
    for b, L in enumerate(lens):
        k[b, :, L:, :] = garbage
        v[b, :, L:, :] = -garbage
    do = f32_to_bf16_bits(_gauss(seed, 3, (B, H, Sq, D)))
    kv_len = np.asarray(lens, np.int32)
    mask = (np.arange(Sk)[None, :] < kv_len[:, None]).astype(np.uint8).reshape(B, 1, 1, Sk)
    return Workload("cfg3_ragged_cross", q, f32_to_bf16_bits(k), f32_to_bf16_bits(v), do,
                    1.0 / math.sqrt(D), kv_len=kv_len, extra={"keep_mask": mask},
                    note="per-sequence key lengths; padded K/V rows hold +-1e4")


def config4(B=1, H=32, S=16384, D=128) -> Workload:
    """Long causal self-attention."""
    seed = SEED_BASE + 4
    m = 1.0 / math.sqrt(2.0)
    t = [f32_to_bf16_bits(_gauss(seed, s, (B, H, S, D), m)) for s in range(4)]
    return Workload("cfg4_long_causal" if S == 16384 else f"cfg4_causal_{S}",
                    t[0], t[1], t[2], t[3], 1.0 / math.sqrt(D), causal=True)


def config5(B=2, H=24, S=4608, D=128, outlier_channel=7, outlier_mul=3.0) -> Workload:
    """SageAttention int8-QK inference forward; K has one 3x outlier channel."""
    seed = SEED_BASE + 5
    q = f32_to_bf16_bits(_gauss(seed, 0, (B, H, S, D)))
    k = _gauss(seed, 1, (B, H, S, D))
    k[..., outlier_channel] *= np.float32(outlier_mul)
    # a non-zero channel mean makes the smoothing step observable
    k[..., outlier_channel] += np.float32(1.5)
    v = f32_to_bf16_bits(_gauss(seed, 2, (B, H, S, D)))
    return Workload("cfg5_sage_int8", q, f32_to_bf16_bits(k), v, None, 1.0 / math.sqrt(D),
                    extra={"qblk": 128, "kblk": 64},
                    note="K channel 7 scaled 3x and shifted +1.5")


CONFIGS = {1: config1, 2: config2, 3: config3, 4: config4, 5: config5}
