"""WQLinear: AWQ GEMM-layout linear module with the reference's constructor and forward.

Mirrors server/text_generation_server/layers/awq/quantize/cuda.py:19-49.  The reference
calls the third-party `awq_inference_engine.gemm_forward_cuda` and refuses to run on ROCm
(gptq/__init__.py:39-43); here the HIP library reads the interleaved-nibble layout
directly, with no conversion to the GPTQ layout.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ... import ops
from ..._lib import LAYOUT_AWQ


class WQLinear(nn.Module):
    def __init__(self, w_bit, group_size, qweight, qzeros, scales, bias: Optional[torch.Tensor]):
        super().__init__()

        if w_bit not in [4]:
            raise NotImplementedError("Only 4-bit are supported for now.")

        self.in_features = qweight.shape[0]
        self.out_features = qweight.shape[1] * 32 // w_bit

        self.w_bit = int(w_bit)
        self.group_size = int(group_size) if group_size != -1 else self.in_features
        # same alignment requirements as the reference (cuda.py:33-35)
        assert self.in_features % self.group_size == 0
        assert self.out_features % (32 // self.w_bit) == 0

        self.qweight = qweight
        self.qzeros = qzeros
        self.scales = scales
        self.bias = bias
        self._packed: Optional[ops.PackedWeight] = None

    def packed(self) -> ops.PackedWeight:
        pk = self._packed
        if pk is None or pk.qweight.data_ptr() != self.qweight.data_ptr():
            pk = ops.make_packed(self.qweight, self.qzeros, self.scales, None, self.group_size, LAYOUT_AWQ)
            self._packed = pk
        return pk

    @torch.no_grad()
    def forward(self, x):
        out_shape = x.shape[:-1] + (self.out_features,)
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype not in (torch.float16, torch.bfloat16):
            x2 = x2.to(torch.float16)
        out = ops.linear(self.packed(), x2, self.bias)
        return out.reshape(out_shape)

    def dequantize(self, dtype: torch.dtype = torch.float16) -> torch.Tensor:
        return ops.dequantize(self.packed(), dtype)
