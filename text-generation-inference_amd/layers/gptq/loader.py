"""Checkpoint -> GPTQWeight: which tensors a quantized linear layer reads and how they
shard.

Mirrors `GPTQWeightsLoader`, server/text_generation_server/layers/gptq/__init__.py:93-445.
The four access patterns differ only in how the three packed tensors are fetched:

  pattern                qweight / scales / qzeros                g_idx (gptq checkpoints)
  get_weights            whole                                    whole, rebased to 0 for exllama
  get_weights_col_packed packed-sharded on dim 1 (q|k|v, gate|up) whole
  get_multi_weights_col  sharded on dim 1, concatenated on dim 1  whole, must agree across prefixes
  get_weights_row        qweight sharded on dim 0; qzeros/scales  sharded on dim 0, rebased with
                         sharded on dim 0 unless act-order or a   the group tables
                         single group keeps them whole

Everything after the fetch is shared (`_finish`): an AWQ checkpoint served with
`--quantize gptq` is repacked to the GPTQ layout (fast_awq_to_gptq) and gets a synthetic
g_idx unless the exllama flag is on.  `use_exllama` keeps the reference's meaning for the
callers that read it; here every flag value reaches the same HIP library.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from ...utils.weights import DefaultWeightsLoader, UnquantizedWeight, Weights, WeightsLoader

_NOT_QUANTIZED = "Cannot load `{}` weight, make sure the model is already quantized"


class GPTQWeightsLoader(WeightsLoader):
    def __init__(
        self,
        *,
        bits: int,
        desc_act: bool,
        groupsize: int,
        quant_method: str,
        quantize: str,
        sym: bool,
        modules_to_not_convert: Optional[List[str]] = None,
    ):
        self.bits = bits
        self.desc_act = desc_act
        self.groupsize = groupsize
        self.quant_method = quant_method
        self.quantize = quantize
        self.sym = sym
        self.modules_to_not_convert = list(modules_to_not_convert or [])
        self._dense = DefaultWeightsLoader(UnquantizedWeight)

    # -- checkpoint conventions -------------------------------------------------------

    @staticmethod
    def is_layer_skipped_quantization(prefix: str, modules_to_not_convert: List[str]) -> bool:
        """A layer stays dense when any listed module name occurs in its prefix
        (gptq/__init__.py:196-199)."""
        return any(module_name in prefix for module_name in modules_to_not_convert)

    def _get_gptq_params(self, weights: Weights) -> None:
        """Checkpoints written by the server's own quantizer carry their settings as
        tensors; they override the JSON-derived ones and imply no act-order
        (gptq/__init__.py:433-445).  Before `gptq_sym` existed that quantizer was always
        asymmetric."""
        if weights.has_tensor("gptq_bits") and weights.has_tensor("gptq_groupsize"):
            self.bits = weights.get_tensor("gptq_bits").item()
            self.groupsize = weights.get_tensor("gptq_groupsize").item()
            self.desc_act = False
            self.sym = weights.get_tensor("gptq_sym").item() if weights.has_tensor("gptq_sym") else False
            self.quant_method = "gptq"

    @property
    def _gptq_checkpoint(self) -> bool:
        return self.quantize == "gptq" and self.quant_method == "gptq"

    @property
    def _awq_as_gptq(self) -> bool:
        return self.quantize == "gptq" and self.quant_method == "awq"

    def _fetch(self, fetch, name: str):
        try:
            return fetch(name)
        except RuntimeError:
            raise RuntimeError(_NOT_QUANTIZED.format(self.quantize))

    def _finish(self, qweight, qzeros, scales, g_idx, use_exllama: bool):
        from . import GPTQWeight

        if self._awq_as_gptq:
            from ..awq.conversion_utils import fast_awq_to_gptq

            qweight, qzeros = fast_awq_to_gptq(qweight, qzeros)
            if use_exllama:
                g_idx = None
            else:
                rows = qweight.shape[0] * (32 // self.bits)
                g_idx = (torch.arange(rows, device=qweight.device) // self.groupsize).to(torch.int32)
        return GPTQWeight(
            qweight=qweight,
            qzeros=qzeros,
            scales=scales,
            g_idx=g_idx,
            bits=self.bits,
            groupsize=self.groupsize,
            use_awq_kernel=self.quantize == "awq",
            use_exllama=use_exllama,
        )

    # -- access patterns --------------------------------------------------------------

    def get_weights(self, weights: Weights, prefix: str):
        """Unsharded layer (gptq/__init__.py:134-194)."""
        self._get_gptq_params(weights)
        if self.is_layer_skipped_quantization(prefix, self.modules_to_not_convert):
            return self._dense.get_weights(weights, prefix)
        use_exllama = self.bits == 4 and not self.desc_act

        qweight = self._fetch(weights.get_tensor, f"{prefix}.qweight")
        g_idx = weights.get_tensor(f"{prefix}.g_idx") if self._gptq_checkpoint else None
        if use_exllama and g_idx is not None:
            g_idx = g_idx - g_idx[0]
        qzeros = weights.get_tensor(f"{prefix}.qzeros")
        scales = weights.get_tensor(f"{prefix}.scales")
        return self._finish(qweight, qzeros, scales, g_idx, use_exllama)

    def get_weights_col_packed(self, weights: Weights, prefix: str, block_sizes):
        """One stored tensor that packs several projections along N
        (gptq/__init__.py:201-260).  The exllama flag is never raised here."""
        if self.is_layer_skipped_quantization(prefix, self.modules_to_not_convert):
            return self._dense.get_weights_col_packed(weights, prefix, block_sizes)

        def packed(name):
            return weights.get_packed_sharded(name, dim=1, block_sizes=block_sizes)

        qweight = self._fetch(packed, f"{prefix}.qweight")
        scales = packed(f"{prefix}.scales").to(dtype=weights.dtype)
        self._get_gptq_params(weights)
        qzeros = packed(f"{prefix}.qzeros")
        g_idx = weights.get_tensor(f"{prefix}.g_idx") if self._gptq_checkpoint else None
        return self._finish(qweight, qzeros, scales, g_idx, use_exllama=False)

    def get_multi_weights_col(self, weights: Weights, prefixes: List[str], dim: int):
        """Several stored layers fused along N (gptq/__init__.py:262-329)."""
        if self.is_layer_skipped_quantization(prefixes[0], self.modules_to_not_convert):
            return self._dense.get_multi_weights_col(weights, prefixes, dim)

        def fused(suffix):
            return torch.cat([weights.get_sharded(f"{p}.{suffix}", dim=1) for p in prefixes], dim=1)

        qweight = self._fetch(fused, "qweight")
        scales = fused("scales")
        self._get_gptq_params(weights)
        qzeros = fused("qzeros")
        use_exllama = self.bits == 4 and self.quantize == "gptq" and not self.desc_act

        g_idx = None
        if self._gptq_checkpoint:
            per_prefix = [weights.get_tensor(f"{p}.g_idx") for p in prefixes]
            for other in per_prefix[1:]:
                torch.testing.assert_close(other, per_prefix[0])
            g_idx = per_prefix[0]
        return self._finish(qweight, qzeros, scales, g_idx, use_exllama)

    def get_weights_row(self, weights: Weights, prefix: str):
        """Layer split along K (gptq/__init__.py:331-431).

        With contiguous groups each rank owns whole groups, so the group tables shard with
        the rows and g_idx is rebased to start at 0.  With act-order (or one group for the
        whole matrix) any row may use any group: the tables stay whole and g_idx keeps
        pointing into them.  A sharded g_idx that is neither `arange // groupsize` (after
        rebasing) nor all zero reveals act-order even when the config did not say so.
        """
        self._get_gptq_params(weights)
        if self.is_layer_skipped_quantization(prefix, self.modules_to_not_convert):
            return self._dense.get_weights_row(weights, prefix)
        use_exllama = self.bits == 4 and not self.desc_act
        desc_act = self.desc_act

        def rows(name):
            return weights.get_sharded(name, dim=0)

        try:
            qweight = rows(f"{prefix}.qweight")
        except RuntimeError:
            raise RuntimeError(
                "Cannot load `gptq` weight, make sure the model is already quantized, or quantize it "
                "with `text-generation-server quantize ORIGINAL_MODEL_ID NEW_MODEL_ID`"
            )
        g_idx = rows(f"{prefix}.g_idx") if self._gptq_checkpoint else None

        if weights.process_group.size() > 1 and g_idx is not None:
            contiguous = torch.arange(g_idx.shape[0], dtype=torch.int32) // int(self.groupsize) \
                if self.groupsize > 0 else torch.zeros(g_idx.shape[0], dtype=torch.int32)
            rebased = (g_idx - g_idx[0]).cpu().to(torch.int32)
            if not torch.equal(rebased, contiguous) and not bool((g_idx == 0).all()):
                use_exllama = False
                desc_act = True

        if not desc_act and self.groupsize != -1:
            qzeros = rows(f"{prefix}.qzeros")
            scales = rows(f"{prefix}.scales")
            if g_idx is not None:
                g_idx = g_idx - g_idx[0]
        else:
            qzeros = weights.get_tensor(f"{prefix}.qzeros")
            scales = weights.get_tensor(f"{prefix}.scales")
        return self._finish(qweight, qzeros, scales, g_idx, use_exllama)
