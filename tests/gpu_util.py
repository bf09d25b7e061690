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
