"""Integer layout helpers between the AWQ and GPTQ checkpoint formats (torch tensors).

Covers what server/text_generation_server/layers/awq/conversion_utils.py:5-97 offers
(pack / unpack / apply_order / fast_awq_to_gptq).  The kernels never need the conversion
(they read both layouts natively); the helpers exist for loaders and tests that want to
move a checkpoint from one layout to the other, and they are pure integer reshuffles.
"""

from __future__ import annotations

from typing import List

import torch

AWQ_PACK_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]
REVERSE_AWQ_PACK_ORDER = [0, 4, 1, 5, 2, 6, 3, 7]

_NIBBLES = 8


def _shifts(device) -> torch.Tensor:
    return torch.arange(0, 32, 4, dtype=torch.int32, device=device)


def pack(imatrix: torch.Tensor, direction: str = "column") -> torch.Tensor:
    """4-bit integers -> int32 words, 8 per word along columns ("column") or rows ("row")."""
    vals = imatrix.to(torch.int32) & 0xF
    sh = _shifts(imatrix.device)
    if direction == "column":
        grouped = vals.reshape(vals.shape[0], vals.shape[1] // _NIBBLES, _NIBBLES)
        words = (grouped << sh.view(1, 1, -1)).sum(dim=-1)
    elif direction == "row":
        grouped = vals.reshape(vals.shape[0] // _NIBBLES, _NIBBLES, vals.shape[1])
        words = (grouped << sh.view(1, -1, 1)).sum(dim=1)
    else:
        raise ValueError(direction)
    # the sum of disjoint nibbles can exceed int32 range only through the sign bit
    return words.to(torch.int32)


def unpack(qmatrix: torch.Tensor, direction: str = "column") -> torch.Tensor:
    """int32 words -> 4-bit integers (int8), inverse of pack()."""
    sh = _shifts(qmatrix.device)
    if direction == "column":
        nib = (qmatrix.unsqueeze(-1) >> sh.view(1, 1, -1)) & 0xF
        out = nib.reshape(qmatrix.shape[0], -1)
    elif direction == "row":
        nib = (qmatrix.unsqueeze(1) >> sh.view(1, -1, 1)) & 0xF
        out = nib.reshape(-1, qmatrix.shape[-1])
    else:
        raise ValueError(direction)
    return out.to(torch.int8)


def apply_order(imatrix: torch.Tensor, direction: str = "column", order: List[int] = AWQ_PACK_ORDER):
    """Permute every block of 8 columns (or rows) by `order`."""
    if direction == "column":
        return imatrix.reshape(-1, _NIBBLES)[:, order].reshape(imatrix.shape)
    if direction == "row":
        return imatrix.reshape(_NIBBLES, -1)[order, :].reshape(imatrix.shape)
    raise ValueError(direction)


def fast_awq_to_gptq(qweight: torch.Tensor, qzeros: torch.Tensor):
    """AWQ (qweight [K, N/8], qzeros [G, N/8]) -> GPTQ (qweight [K/8, N], qzeros [G, N/8]).

    Un-interleave the nibbles, store zero points minus one (the GPTQ reader adds one),
    pack weights along rows and zero points along columns.
    """
    izeros = apply_order(unpack(qzeros, "column"), "column", REVERSE_AWQ_PACK_ORDER)
    iweights = apply_order(unpack(qweight, "column"), "column", REVERSE_AWQ_PACK_ORDER)
    return pack(iweights, "row"), pack(izeros - 1, "column")
