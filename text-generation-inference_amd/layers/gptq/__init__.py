"""GPTQ / AWQ weight container and its dispatch to the MI355X linear modules.

Mirrors server/text_generation_server/layers/gptq/__init__.py:18-90 (GPTQWeight) and
:448-479 (the exllama exports).  Every branch ends in the same HIP library; the three
module classes only differ in the constructor signature the reference callers expect.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .quant_linear import QuantLinear  # noqa: F401
from .exllama import (  # noqa: F401
    ExllamaQuantLinear,
    create_exllama_buffers,
    set_device,
)
from .loader import GPTQWeightsLoader  # noqa: F401

# The reference sets this to "1"/"2" when an exllama extension imported; here the native
# library always plays that role.
HAS_EXLLAMA = "2"
CAN_EXLLAMA = True


@dataclass
class GPTQWeight:
    """Tensors of one quantized linear layer, exactly as the loaders hand them over."""

    qweight: torch.Tensor
    qzeros: torch.Tensor
    scales: torch.Tensor
    g_idx: Optional[torch.Tensor]
    bits: int
    groupsize: int
    use_awq_kernel: bool
    use_exllama: bool

    def __post_init__(self):
        # gptq/__init__.py:29-31: fp32 scales are narrowed once, at construction
        if self.scales.dtype == torch.float:
            self.scales = self.scales.half()

    @property
    def device(self) -> torch.device:
        return self.qweight.device

    def get_linear(self, bias: Optional[torch.Tensor]):
        if self.use_awq_kernel:
            # The reference refuses this branch on ROCm (gptq/__init__.py:39-43); the
            # native kernel consumes the AWQ GEMM layout directly.
            from ..awq.quantize import WQLinear

            return WQLinear(
                w_bit=self.bits,
                group_size=self.groupsize,
                qweight=self.qweight,
                qzeros=self.qzeros,
                scales=self.scales,
                bias=bias,
            )
        if self.use_exllama:
            return ExllamaQuantLinear(self, bias)
        return QuantLinear(
            self.qweight,
            self.qzeros,
            self.scales,
            self.g_idx,
            bias,
            self.bits,
            self.groupsize,
        )
