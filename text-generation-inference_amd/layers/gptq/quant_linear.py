"""QuantLinear: the GPTQ linear module with the reference's constructor and forward.

Mirrors server/text_generation_server/layers/gptq/triton.py:252-292,351-363: same
positional constructor, same attributes (qweight, qzeros, scales, g_idx, bias, bits,
maxq, groupsize, infeatures, outfeatures), same `new()` factory, same forward contract
(any leading dims, reshape to [-1, K], bias added after, reshape back).  The matmul is
the HIP library's q4_linear instead of the Triton kernel.
"""

from __future__ import annotations

import math
import os
from typing import Optional

import numpy as np
import torch
import torch.nn as nn

from ... import ops
from ..._lib import LAYOUT_GPTQ


# Act-order layers: "table" (default) runs the kernels that read the checkpoint layout and look
# every row's group up through g_idx; nothing is repacked.  "repack" opts into what the
# reference's exllama matrices do at load time (QMatrix::make_sequential): a second qweight with
# the rows in group order, kept privately next to the checkpoint tensor (twice the weight
# memory), served by the contiguous-group kernels, which are faster at decode.
ACT_ORDER_MODE = os.environ.get("Q4_ACT_ORDER", "table")


def is_trivial_g_idx(g_idx: torch.Tensor, groupsize: int) -> bool:
    """True when g_idx is the sequential map k -> k // groupsize (no activation order).

    The same test the reference's exllama wrappers run at construction
    (gptq/exllama.py:81-92: all zeros, or equal to [i // groupsize]); it runs once per
    layer at load time, so the device->host sync it implies is outside the forward path.
    """
    K = g_idx.numel()
    if K == 0:
        return True
    gs = K if groupsize == -1 else int(groupsize)
    expect = torch.arange(K, device=g_idx.device, dtype=torch.int64) // gs
    return bool(torch.equal(g_idx.to(torch.int64), expect))


class QuantLinear(nn.Module):
    def __init__(self, qweight, qzeros, scales, g_idx, bias, bits, groupsize):
        super().__init__()
        self.register_buffer("qweight", qweight)
        self.register_buffer("qzeros", qzeros)
        self.register_buffer("scales", scales)
        self.register_buffer("g_idx", g_idx)
        if bias is not None:
            self.register_buffer("bias", bias)
        else:
            self.bias = None
        if bits not in [4]:
            raise NotImplementedError("Only 4 bits are supported.")
        self.bits = int(bits)
        self.maxq = 2**self.bits - 1
        self.groupsize = int(groupsize)

        self.outfeatures = qweight.shape[1]
        self.infeatures = qweight.shape[0] * 32 // self.bits
        self._packed: Optional[ops.PackedWeight] = None
        self._packed_of = None  # data pointer of the qweight the kernel view was built from
        if qweight is not None and qweight.is_cuda:
            self.post_init()

    @classmethod
    def new(cls, bits, groupsize, infeatures, outfeatures, bias):
        """Zero-filled layer of the given geometry (triton.py:272-292)."""
        if bits not in [4]:
            raise NotImplementedError("Only 4 bits are supported.")
        gs = infeatures if groupsize == -1 else groupsize
        groups = math.ceil(infeatures / gs)
        qweight = torch.zeros((infeatures // 32 * bits, outfeatures), dtype=torch.int32)
        qzeros = torch.zeros((groups, outfeatures // 32 * bits), dtype=torch.int32)
        scales = torch.zeros((groups, outfeatures), dtype=torch.float16)
        g_idx = (torch.arange(infeatures, dtype=torch.int64) // gs).to(torch.int32)
        bias_t = torch.zeros((outfeatures,), dtype=torch.float16) if bias else None
        return cls(qweight, qzeros, scales, g_idx, bias_t, bits, groupsize)

    def pack(self, linear, scales, zeros, g_idx=None):
        """Quantize a dense layer into this module's packed buffers (triton.py:294-349).

        `linear.weight` is [outfeatures, infeatures]; `scales` and `zeros` are
        [outfeatures, groups] as a GPTQ quantizer emits them.  Row k of the integer
        matrix is round((W[:, k] + zero*scale) / fp16(scale)) with its group's
        parameters (round half to even); eight consecutive rows fill one qweight word
        from the low nibble up, eight consecutive columns one qzeros word, and the
        stored zero point is zero - 1.  Like the reference, nothing is clamped: the
        quantizer is expected to hand in weights that land on 0..15 and zeros in 1..16.
        Runs on the CPU at conversion time; the caller moves the module afterwards.
        """
        if g_idx is not None:
            self.g_idx = g_idx.clone()
        gi = self.g_idx.to(torch.int64).cpu()
        scales = scales.detach().cpu().t().contiguous()
        zeros = zeros.detach().cpu().t().contiguous()
        scale_zeros = zeros * scales
        self.scales = scales.clone().half()
        if getattr(linear, "bias", None) is not None:
            self.bias = linear.bias.detach().clone().half()

        w = linear.weight.detach().cpu().t()  # [K, N]
        q = torch.round((w + scale_zeros[gi]) / self.scales[gi]).to(torch.int32)
        per_word = 32 // self.bits
        shifts = (np.arange(per_word, dtype=np.uint32) * np.uint32(self.bits))
        qi = q.numpy().astype(np.uint32).reshape(-1, per_word, q.shape[1])
        qweight = np.bitwise_or.reduce(qi << shifts[None, :, None], axis=1)
        self.qweight = torch.from_numpy(qweight.astype(np.int32))

        z = (zeros - 1).to(torch.int64).numpy().astype(np.uint32)  # -1 wraps to all ones
        zi = z.reshape(z.shape[0], -1, per_word)
        qzeros = np.bitwise_or.reduce(zi << shifts[None, None, :], axis=2)
        self.qzeros = torch.from_numpy(qzeros.astype(np.int32))
        self._packed = None

    def post_init(self) -> ops.PackedWeight:
        """The load-time work of the layer (the reference's exllama modules do theirs in
        post_init at Warmup, exllamav2.py:215-224): the act-order test on g_idx (one
        device->host sync), validation, the optional row reorder, the launch plans of the
        decode sizes and the workspace.  The registered buffers are never written: a
        state_dict saved afterwards is still the checkpoint."""
        g_idx = self.g_idx
        if g_idx is not None and is_trivial_g_idx(g_idx, self.groupsize):
            g_idx = None  # sequential groups: the kernels index by k // groupsize
        pk = ops.make_packed(self.qweight, self.qzeros, self.scales, g_idx, self.groupsize, LAYOUT_GPTQ)
        if pk.g_idx is not None and ACT_ORDER_MODE == "repack" and self.qweight.is_cuda:
            seq = ops.make_sequential(pk)
            if seq is not None:
                pk = seq
        pk.prepare()
        self._packed = pk
        self._packed_of = self.qweight.data_ptr()
        return pk

    def packed(self) -> ops.PackedWeight:
        """Kernel view of the buffers, rebuilt if they moved (e.g. `.to(device)`) or were
        rewritten (`pack`)."""
        pk = self._packed
        if pk is None or self._packed_of != self.qweight.data_ptr():
            pk = self.post_init()
        return pk

    @torch.no_grad()
    def forward(self, x):
        out_shape = x.shape[:-1] + (self.outfeatures,)
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype not in (torch.float16, torch.bfloat16):
            x2 = x2.to(torch.float16)  # the reference computes this path in fp16 (triton.py:246)
        out = ops.linear(self.packed(), x2, self.bias)
        return out.reshape(out_shape)

    def dequantize(self, dtype: torch.dtype = torch.float16) -> torch.Tensor:
        """Dense [K, N] weight, bit-exact with the reference's dequantize step."""
        return ops.dequantize(self.packed(), dtype)
