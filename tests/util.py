"""Helpers shared by the tests."""
import numpy as np
import torch


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16).copy()).view(torch.bfloat16)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.detach().float().cpu()
    b = b.detach().float().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


FINITE_BF16 = np.concatenate([np.arange(0, 0x7F80), np.arange(0x8000, 0xFF80)]).astype(np.uint16)
ALL_POS_FINITE = np.arange(0, 0x7F80, dtype=np.uint16)


def bf16_ulps(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """distance in bf16 steps between two bf16 tensors (sign-magnitude ordering)"""
    ia = a.detach().cpu().contiguous().view(torch.int16).to(torch.int32)
    ib = b.detach().cpu().contiguous().view(torch.int16).to(torch.int32)
    ia = torch.where(ia < 0, -(ia & 0x7fff), ia)
    ib = torch.where(ib < 0, -(ib & 0x7fff), ib)
    return (ia - ib).abs()
