"""Entry of the hot path: get_linear(weight, bias) -> module.

Mirrors server/text_generation_server/layers/linear.py:116-126 for quantization-aware
weights: anything that knows how to build its own linear layer does so.  Bare tensors
(unquantized weights) are not part of this package.
"""

from __future__ import annotations

import torch


def get_linear(weight, bias):
    if isinstance(weight, torch.Tensor):
        raise NotImplementedError(
            "unquantized linear layers are outside this package; pass a GPTQWeight"
        )
    return weight.get_linear(bias)
