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


def fold_down_permutation(gate_up_layer, down_layer) -> bool:
    """Remove the run-time activation gather of an act-order down projection.

    A down projection whose rows were put into group order reads its input through a
    permutation (x_seq[:, j] = x[:, perm[j]]).  Its input is act(gate) * up, element by element,
    so the permutation can be applied once, at load time, to the output columns of the gate and
    the up half of the gate_up projection instead: the first half of the MLP then produces its
    result directly in the order the down projection's rows are in, and the down projection
    becomes a plain contiguous-group layer.  Only the layers' private kernel views (and the
    gate_up bias) change; the checkpoint tensors they were built from stay as they are.  Both
    layers must come from this package; returns False (nothing changed) when the down projection
    has no permutation (the default: rows stay in checkpoint order unless Q4_ACT_ORDER=repack) or
    the shapes do not pair up.  Afterwards `down_layer.dequantize()` returns its matrix with the rows in group
    order, the one that multiplies the reordered activations."""
    gpk = gate_up_layer.packed() if callable(getattr(gate_up_layer, "packed", None)) else gate_up_layer._packed
    dpk = down_layer.packed() if callable(getattr(down_layer, "packed", None)) else down_layer._packed
    if dpk.perm is None or gpk.layout != ops.LAYOUT_GPTQ or gpk.N != 2 * dpk.K:
        return False
    inter = dpk.K
    perm = dpk.perm.to(torch.int64)
    cols = torch.cat([perm, perm + inter])
    new = ops.permute_output_columns(gpk, cols)
    bias = getattr(gate_up_layer, "bias", None)
    if bias is not None:
        gate_up_layer.bias = bias.index_select(0, cols.to(bias.device))
    gate_up_layer._packed = new
    plain = ops.PackedWeight(dpk.qweight, dpk.qzeros, dpk.scales, None, dpk.K, dpk.N, dpk.groupsize,
                             dpk.num_groups, dpk.layout)
    new.prepare()
    plain.prepare()
    down_layer._packed = plain
    return True
