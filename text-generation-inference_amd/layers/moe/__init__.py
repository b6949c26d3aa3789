"""Sparse mixture-of-experts layer on GPTQ int4 experts.

Mirrors the constructor and forward of the reference's `GPTQMarlinSparseMoELayer`
(server/text_generation_server/layers/moe/gptq_marlin.py:54-146): the experts' gate/up and
down projections are loaded through the same `Weights` calls (`get_multi_weights_col`,
`get_weights_row`, :149-183) and stacked along a leading expert dimension (:186-229), and
`forward(x, gating_output=...)` routes every token to its top-k experts.  Differences: the
tensors stay in checkpoint layout -- GPTQ with or without act-order, or AWQ (no Marlin repack,
hence no perm / is_full_k fields) -- and
the grouped int4 kernels of this package do the work that the reference takes from the
`kernels-community/moe` package, which only exists for CUDA.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn as nn

from ... import ops
from ..._lib import LAYOUT_AWQ, LAYOUT_GPTQ
from ..gptq import GPTQWeight
from ..awq.conversion_utils import fast_awq_to_gptq
import os

from ..gptq.quant_linear import is_trivial_g_idx

# The expert weights keep the load-time conversions as their default (the reference's MoE layer
# repacks every expert into the Marlin layout when it is built, layers/moe/gptq_marlin.py:186-229):
# AWQ-layout experts go to the GPTQ layout once, act-order experts get their rows put into
# group order.  "native" / "table" keep the checkpoint layout and run the AWQ / lookup kernels.
AWQ_MODE = os.environ.get("Q4_MOE_AWQ", "convert")
ACT_ORDER_MODE = os.environ.get("Q4_MOE_ACT_ORDER", "repack")


@dataclass
class GPTQMoEWeight:
    """Stacked experts of one projection: qweight [E, K/8, N] (AWQ: [E, K, N/8]), qzeros
    [E, G, N/8], scales [E, G, N], g_idx [E, K] or None."""

    qweight: torch.Tensor
    qzeros: torch.Tensor
    scales: torch.Tensor
    g_idx: Optional[torch.Tensor]
    groupsize: int
    use_awq_kernel: bool

    q_perm: Optional[torch.Tensor] = None  # set once the experts' rows are in group order
    # rows in group order with the activations' order folded into the producer's columns:
    # plain contiguous-group experts, g_idx no longer describes the stored rows
    rows_in_group_order: bool = False

    def packed(self) -> ops.PackedMoeWeight:
        if self.use_awq_kernel and AWQ_MODE != "native" and self.qweight.is_cuda:
            # AWQ-layout experts: one conversion to the GPTQ layout (bit-exact, see WQLinear),
            # expert by expert to bound the temporaries; the AWQ tensors are dropped
            converted = [fast_awq_to_gptq(self.qweight[e], self.qzeros[e]) for e in range(self.qweight.shape[0])]
            self.qweight = torch.stack([c[0] for c in converted]).contiguous()
            self.qzeros = torch.stack([c[1] for c in converted]).contiguous()
            self.use_awq_kernel = False
        g_idx = self.g_idx
        if self.rows_in_group_order or self.q_perm is not None or (
                g_idx is not None and all(is_trivial_g_idx(g, self.groupsize) for g in g_idx)):
            g_idx = None  # sequential groups in every expert: the kernels index by k // groupsize
        pk = ops.make_packed_moe(self.qweight, self.qzeros, self.scales, self.groupsize, g_idx,
                                 LAYOUT_AWQ if self.use_awq_kernel else LAYOUT_GPTQ)
        if self.q_perm is not None:
            pk.perm = self.q_perm
        elif g_idx is not None and ACT_ORDER_MODE != "table" and self.qweight.is_cuda:
            # act-order experts: rows into group order once, like the dense layers; the
            # checkpoint-order tensor is dropped
            seq = ops.make_sequential_moe(pk)
            if seq is not None:
                self.qweight = seq.qweight
                self.q_perm = seq.perm
                pk = seq
        return pk


def _check_expert(weight, name: str) -> GPTQWeight:
    if not isinstance(weight, GPTQWeight):
        raise ValueError(f"{name}: expected GPTQ weights, got {type(weight).__name__}")
    if weight.bits != 4:
        raise NotImplementedError(f"{name}: only 4-bit experts are supported, got {weight.bits}")
    return weight


def _pack_weight(*, n_experts: int, expert: int, moe_weight: Optional[GPTQMoEWeight], weight: GPTQWeight) -> GPTQMoEWeight:
    """gptq_marlin.py:186-229: allocate on the first expert, copy every expert into its slice."""
    if moe_weight is None:
        moe_weight = GPTQMoEWeight(
            qweight=torch.empty((n_experts,) + weight.qweight.shape, dtype=weight.qweight.dtype, device=weight.qweight.device),
            qzeros=torch.empty((n_experts,) + weight.qzeros.shape, dtype=weight.qzeros.dtype, device=weight.qzeros.device),
            scales=torch.empty((n_experts,) + weight.scales.shape, dtype=weight.scales.dtype, device=weight.scales.device),
            g_idx=None if weight.g_idx is None else torch.empty(
                (n_experts,) + weight.g_idx.shape, dtype=weight.g_idx.dtype, device=weight.g_idx.device),
            groupsize=weight.groupsize,
            use_awq_kernel=weight.use_awq_kernel,
        )
    if weight.groupsize != moe_weight.groupsize or weight.use_awq_kernel != moe_weight.use_awq_kernel:
        raise ValueError(f"expert {expert} differs from expert 0 in groupsize or layout")
    if (weight.g_idx is None) != (moe_weight.g_idx is None):
        raise ValueError(f"expert {expert} differs from expert 0 in having a g_idx")
    moe_weight.qweight[expert] = weight.qweight
    moe_weight.qzeros[expert] = weight.qzeros
    moe_weight.scales[expert] = weight.scales
    if weight.g_idx is not None:
        moe_weight.g_idx[expert] = weight.g_idx
    return moe_weight


def _load_expert_multi_weights_col(*, prefix: str, n_experts: int, names: List[str], weights) -> GPTQMoEWeight:
    moe_weight = None
    for i in range(n_experts):
        weight = weights.get_multi_weights_col([f"{prefix}.{i}.{name}" for name in names], 0)
        moe_weight = _pack_weight(n_experts=n_experts, expert=i, moe_weight=moe_weight,
                                  weight=_check_expert(weight, f"{prefix}.{i}"))
    assert moe_weight is not None
    return moe_weight


def _load_expert_weights_row(*, prefix: str, n_experts: int, name: str, weights) -> GPTQMoEWeight:
    moe_weight = None
    for i in range(n_experts):
        weight = weights.get_weights_row(f"{prefix}.{i}.{name}")
        moe_weight = _pack_weight(n_experts=n_experts, expert=i, moe_weight=moe_weight,
                                  weight=_check_expert(weight, f"{prefix}.{i}.{name}"))
    assert moe_weight is not None
    return moe_weight


class GPTQSparseMoELayer(nn.Module):
    """MoE layer on the grouped int4 kernels; same keyword constructor as the reference's."""

    def __init__(
        self,
        *,
        n_expert_group: Optional[int],
        n_experts: int,
        prefix: str,
        renormalize: bool,
        topk: int,
        topk_group: Optional[int],
        weights,
        gate_proj_name: str = "gate_proj",
        up_proj_name: str = "up_proj",
        down_proj_name: str = "down_proj",
        scoring_func: Optional[str] = "softmax",
        e_score_correction_bias: Optional[float] = None,
        hidden_act: str = "silu",
    ):
        super().__init__()
        assert (n_expert_group is None) == (
            topk_group is None
        ), "n_expert_group and topk_group must both be None or have some value"
        if scoring_func not in (None, "softmax"):
            raise NotImplementedError(f"scoring func {scoring_func} is not handled")
        if e_score_correction_bias is not None:
            raise NotImplementedError("e_score_correction_bias is not implemented")
        self.n_experts = n_experts
        self.n_expert_group = n_expert_group
        self.topk_group = topk_group
        self.topk = topk
        self.renormalize = renormalize
        self.hidden_act = hidden_act
        self.gate_up_proj = _load_expert_multi_weights_col(
            prefix=prefix, n_experts=n_experts, names=[gate_proj_name, up_proj_name], weights=weights
        )
        self.down_proj = _load_expert_weights_row(prefix=prefix, n_experts=n_experts, name=down_proj_name, weights=weights)
        self.bits = 4
        self._gate_up = self.gate_up_proj.packed()
        self._down = self.down_proj.packed()
        # act-order experts: the second projection's input order goes into the first one's
        # output columns, expert by expert (no activation gather between the projections)
        folded_gate_up, folded_down = ops.fold_moe_down_permutation(self._gate_up, self._down)
        if folded_down is not self._down:
            self.gate_up_proj.qweight, self.gate_up_proj.qzeros, self.gate_up_proj.scales = (
                folded_gate_up.qweight, folded_gate_up.qzeros, folded_gate_up.scales)
            self.down_proj.q_perm = None
            self.down_proj.rows_in_group_order = True
            self._gate_up, self._down = folded_gate_up, folded_down

    @torch.no_grad()
    def forward(self, x: torch.Tensor, *, gating_output: torch.Tensor) -> torch.Tensor:
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        assert x2.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
        assert gating_output.shape[1] == self.n_experts, "Number of experts mismatch"
        out = ops.moe_forward(self._gate_up, self._down, x2, gating_output, self.topk, self.renormalize, self.hidden_act,
                              self.n_expert_group or 0, self.topk_group or 0)
        return out.reshape(shape)
