"""WQLinear: AWQ GEMM-layout linear module with the reference's constructor and forward.

Mirrors server/text_generation_server/layers/awq/quantize/cuda.py:19-49.  The reference
calls the third-party `awq_inference_engine.gemm_forward_cuda` and refuses to run on ROCm
(gptq/__init__.py:39-43); here the HIP kernels read the interleaved-nibble layout as it
sits in the checkpoint: nothing is repacked and `qweight` / `qzeros` / `scales` stay the
tensors the loader handed in.

Q4_AWQ=convert opts into the reference's own route for AWQ checkpoints on ROCm
(fast_awq_to_gptq, gptq/__init__.py:186-204): one conversion to the GPTQ layout at load time,
kept in private tensors next to the checkpoint ones (twice the weight memory), served by the
GPTQ kernels, which are faster at decode.  The two routes compute the same weights bit for
bit: the GPTQ reader's +1 undoes the -1 of the conversion for every zero point, 0 included
(15 + 1 wraps to 0).
"""

from __future__ import annotations

import os
from typing import Optional

import torch
import torch.nn as nn

from ... import ops
from ..._lib import LAYOUT_AWQ, LAYOUT_GPTQ
from .conversion_utils import fast_awq_to_gptq

# "native": the AWQ-layout kernels on the checkpoint tensors; "convert": GPTQ-layout copy + GPTQ kernels
AWQ_MODE = os.environ.get("Q4_AWQ", "native")


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
        self._packed_of = None  # data pointer of the qweight the kernel view was built from
        if qweight.is_cuda:
            self.post_init()

    def post_init(self) -> ops.PackedWeight:
        """Everything that is not the matmul happens here, once, when the tensors are on the GPU:
        validation, the optional layout conversion, the launch plans of the decode sizes and the
        workspace.  The forward is then one library call."""
        if AWQ_MODE == "convert" and self.qweight.is_cuda:
            gq, gz = fast_awq_to_gptq(self.qweight, self.qzeros)
            pk = ops.make_packed(gq.contiguous(), gz.contiguous(), self.scales, None, self.group_size, LAYOUT_GPTQ)
        else:
            pk = ops.make_packed(self.qweight, self.qzeros, self.scales, None, self.group_size, LAYOUT_AWQ)
        pk.prepare()
        self._packed = pk
        self._packed_of = self.qweight.data_ptr()
        return pk

    def packed(self) -> ops.PackedWeight:
        """Kernel view of the tensors, rebuilt if they were replaced (e.g. moved to a device)."""
        pk = self._packed
        if pk is None or self._packed_of != self.qweight.data_ptr():
            pk = self.post_init()
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
