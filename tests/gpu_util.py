"""Helpers shared by the GPU parity tests: numpy <-> device tensors."""
import numpy as np
import torch


def dev_i8(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int8)).cuda()


def dev_bf16(bits: np.ndarray) -> torch.Tensor:
    """uint16 bf16 bit patterns -> torch.bfloat16 tensor on the GPU."""
    t = torch.from_numpy(np.ascontiguousarray(bits, dtype=np.uint16).view(np.int16).copy())
    return t.view(torch.bfloat16).cuda()


def host_bits(t: torch.Tensor) -> np.ndarray:
    """torch.bfloat16 tensor -> uint16 bit patterns (numpy)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def bf16_ulp_distance(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in units of bf16 steps between two arrays of bit patterns
    (sign-magnitude mapped to a monotone integer line)."""

    def mono(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)

    return np.abs(mono(a_bits) - mono(b_bits))
