"""Shared helpers of the parity tests: oracle arrays <-> device tensors, error metrics."""

from __future__ import annotations

import numpy as np
import torch


def to_dev(a, device, bf16=False):
    """NumPy array -> device tensor (uint16 bf16 bit patterns become torch.bfloat16)."""
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16 and bf16:
        return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).to(device)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).to(device)


def bits_of(t: torch.Tensor) -> np.ndarray:
    """Raw 16-bit patterns of an fp16/bf16 tensor."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def to_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def max_rel_err(y: np.ndarray, ref: np.ndarray) -> float:
    """max|y - ref| / max|ref|: the parity bar's metric (outputs are zero-mean, so an
    element-wise ratio would blow up near zero crossings)."""
    denom = float(np.max(np.abs(ref)))
    if denom == 0.0:
        return float(np.max(np.abs(y)))
    return float(np.max(np.abs(y.astype(np.float64) - ref.astype(np.float64))) / denom)
