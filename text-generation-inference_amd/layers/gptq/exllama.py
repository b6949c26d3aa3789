"""ExllamaQuantLinear: the handle-free equivalent of the reference's exllama modules.

Mirrors the constructor `(weight: GPTQWeight, bias)` and forward of
server/text_generation_server/layers/gptq/exllamav2.py:178-231 and
gptq/exllama.py:66-134.  The reference needs a Warmup hook (`set_device`,
`create_exllama_buffers`, server.py:103-116) to allocate a dequant scratch buffer and to
repack qweight in place; nothing of that exists here (the kernels read the checkpoint
layout and never materialise W).  `set_device` is kept as a no-op for call compatibility;
`create_exllama_buffers(max_total_tokens)`, which the server calls once after the model is
loaded and before it captures its decode graphs, is where this package does its own one-time
work over all layers: the shared workspace is sized for `max_total_tokens` rows and the decode
launch plans are measured (`ops.autotune`; `Q4_AUTOTUNE=0` keeps the library's fitted choices).
"""

from __future__ import annotations

import os

import torch
import torch.nn as nn

from ... import ops
from ..._lib import LAYOUT_GPTQ
from . import quant_linear
from .quant_linear import is_trivial_g_idx

DEVICE = None


def set_device(device):
    """Kept for call compatibility (exllamav2.py:154-156); the library holds no device state."""
    global DEVICE
    DEVICE = device


def create_exllama_buffers(max_total_tokens: int = 4096):
    """The reference's Warmup hook (exllamav2.py:159-175: scratch sized for max_total_tokens,
    device matrices built).  Here: every layer built so far fetches its launch plans up to
    `max_total_tokens` rows and the shared workspace grows to the largest need, then the decode
    plans of all layers are measured on the GPU (one pass per distinct layer shape; the report is
    kept in `ops.last_autotune_report`).  Returns None, like the reference's hook."""
    weights = [r() for r in ops._prepared]
    weights = [w for w in weights if w is not None and w.qweight.is_cuda]
    for w in weights:
        w.prepare(max_rows=int(max_total_tokens))
    if weights and os.environ.get("Q4_AUTOTUNE", "1") != "0":
        ops.autotune(weights)
    return None


class ExllamaQuantLinear(nn.Module):
    QUANT_TYPE = "q4-mi355x"

    def __init__(self, weight, bias):
        super().__init__()
        if weight.bits != 4:
            raise ValueError(
                f"The int4 kernels support only bits=4, requested bits={weight.bits}. "
                "Something is wrong in the model initialization."
            )
        self.q_tensors = weight
        self.infeatures = weight.qweight.shape[0] // weight.bits * 32
        self.outfeatures = weight.qweight.shape[1]
        self.device = weight.device
        self.bias = bias if bias is not None else None
        g_idx = weight.g_idx
        # act-order only if g_idx is a real permutation (exllamav2.py:106, exllama.py:81-92)
        if g_idx is not None and (
            bool((g_idx == 0).all()) or is_trivial_g_idx(g_idx, weight.groupsize)
        ):
            g_idx = None
        if g_idx is not None:
            # The exllama kernels only look at the *order* of g_idx (rows are sorted by it and
            # group i of the sorted rows is i // groupsize: exllamav2.py:106-130 -> make_sequential,
            # q_matrix.cu:566-650), and the loader hands this module `g_idx - g_idx[0]`
            # (gptq/__init__.py:163-164, 395-397), whose smallest entry is negative whenever row 0
            # is not in the first group.  The kernels here index the scale / zero tables with
            # g_idx itself, so it is rebased to start at 0: the same groups exllama would form.
            g_idx = g_idx - g_idx.min()
        self.act_order = g_idx is not None
        groupsize = weight.groupsize
        if g_idx is None and weight.scales.shape[0] == 1:
            groupsize = self.infeatures
        # The reference shuffles q_weight in place when it builds its matrix (exllamav2.py:106-130
        # -> make_q_matrix -> QMatrix::make_sequential); here the checkpoint tensors are read as
        # they are.  With Q4_ACT_ORDER=repack a second qweight with the rows in group order is
        # kept privately and the weight object stays untouched.
        pk = ops.make_packed(weight.qweight, weight.qzeros, weight.scales, g_idx, groupsize, LAYOUT_GPTQ)
        if self.act_order and quant_linear.ACT_ORDER_MODE == "repack" and weight.qweight.is_cuda:
            seq = ops.make_sequential(pk)
            if seq is not None:
                pk = seq
        pk.prepare()
        self._packed = pk

    def post_init(self, temp_dq=None):
        """The reference builds its device matrix here at Warmup (exllamav2.py:215-224); this
        module has done its load-time work in the constructor."""
        return None

    @torch.no_grad()
    def forward(self, x, force_cuda=False):
        out_shape = x.shape[:-1] + (self.outfeatures,)
        x2 = x.reshape(-1, x.shape[-1])
        if x2.dtype not in (torch.float16, torch.bfloat16):
            raise TypeError(f"x must be float16 (or bfloat16), got {x2.dtype}")  # ext.cpp:110
        out = ops.linear(self._packed, x2, self.bias)
        return out.reshape(out_shape)

    def dequantize(self, dtype: torch.dtype = torch.float16) -> torch.Tensor:
        return ops.dequantize(self._packed, dtype)
