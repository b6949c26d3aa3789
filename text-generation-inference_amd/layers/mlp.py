"""First half of a gated MLP on a quantized gate_up projection.

The reference computes `gate_up_proj(x)`, views the result as [M, 2, I] and forms
`act(gate) * up` with separate elementwise kernels
(server/text_generation_server/models/custom_modeling/flash_llama_modeling.py:400-404); it
fuses the three only for unquantized fp16 decode on ROCm (`ops.LLMM_Silu`, :378-397).  Here
the activation and the product are the epilogue of the int4 kernels, so the [M, 2I]
intermediate never reaches HBM.  An MLP module switches over by replacing

    gate_up = self.gate_up_proj(x); h = self.act(gate_up[:, 0]) * gate_up[:, 1]

with `h = gate_up_act(self.gate_up_proj, x, self.hidden_act)`.
"""

from __future__ import annotations

import torch

from .. import ops


def gate_up_act(layer, x: torch.Tensor, hidden_act: str = "silu") -> torch.Tensor:
    """`layer` is any module of this package built from a [gate | up] weight
    (QuantLinear, ExllamaQuantLinear, WQLinear); returns act(gate) * up, [..., N/2]."""
    packed = layer.packed() if callable(getattr(layer, "packed", None)) else layer._packed
    x2 = x.reshape(-1, x.shape[-1])
    if x2.dtype not in (torch.float16, torch.bfloat16):
        x2 = x2.to(torch.float16)
    out = ops.linear_gate_up(packed, x2, hidden_act, getattr(layer, "bias", None))
    return out.reshape(x.shape[:-1] + (packed.N // 2,))
