"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor (any device) -> uint16 numpy bit patterns."""
    return t.detach().cpu().contiguous().view(torch.uint16).numpy().copy()


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).copy()).view(torch.bfloat16)


def u8(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().copy()


def rel_fro(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.double(), want.double()
    return float((got - want).norm() / want.norm())


def max_abs(got, want) -> float:
    return float((torch.as_tensor(got).double() - torch.as_tensor(want).double()).abs().max())
