"""PyTorch-on-CPU restatement of the reference's dequantize-then-matmul path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE: only tests/ and bench.py's cpu_baseline leg
import it (the product path is the HIP library and never comes here).

Same arithmetic as q4_oracle.py (NumPy), written with the tensor idiom the reference's own
pure-PyTorch code uses (unpack with broadcast shifts and a mask, then `x.float() @ W.float()`):
  backends/gaudi/server/text_generation_server/layers/gptq/hpu.py:58-78,197-204 (GPTQ),
  backends/gaudi/server/text_generation_server/layers/awq/quantize/hpu.py:22-72,126-134 (AWQ),
  server/text_generation_server/layers/gptq/triton.py:184-192 (the +1 on stored zero points),
  server/text_generation_server/layers/awq/conversion_utils.py:5-6 (AWQ nibble order).
It exists so that the CPU baseline runs on every host core through torch's thread pool, as the
baseline plan states.  Pinned by tests/test_oracle.py::test_torch_restatement_matches_numpy_oracle:
bit-exact dequantized weights and identical fp32 outputs against q4_oracle.py, which is itself
pinned by known answers (see its header).
"""

from __future__ import annotations

import torch

_SHIFTS = torch.arange(0, 32, 4, dtype=torch.int32)
_AWQ_REVERSE = torch.tensor([0, 4, 1, 5, 2, 6, 3, 7], dtype=torch.int64)  # conversion_utils.py:6


def unpack_rows(qmatrix: torch.Tensor) -> torch.Tensor:
    """int32 [R, C] -> int32 [8R, C]: nibble j of word [r, c] is element [8r+j, c] (triton.py:160-169)."""
    out = (qmatrix[:, None, :] >> _SHIFTS[None, :, None]) & 0xF
    return out.reshape(qmatrix.shape[0] * 8, qmatrix.shape[1])


def unpack_cols(qmatrix: torch.Tensor) -> torch.Tensor:
    """int32 [R, C] -> int32 [R, 8C]: nibble j of word [r, c] is element [r, 8c+j] (triton.py:167,184)."""
    out = (qmatrix[:, :, None] >> _SHIFTS[None, None, :]) & 0xF
    return out.reshape(qmatrix.shape[0], qmatrix.shape[1] * 8)


def awq_unpack_cols(qmatrix: torch.Tensor) -> torch.Tensor:
    """AWQ words: position p holds column 8c + [0,2,4,6,1,3,5,7][p] (conversion_utils.py:35-58)."""
    flat = unpack_cols(qmatrix).reshape(qmatrix.shape[0], -1, 8)
    return flat[:, :, _AWQ_REVERSE].reshape(qmatrix.shape[0], -1)


def dequant_gptq(qweight, qzeros, scales, g_idx=None, groupsize=128) -> torch.Tensor:
    """fp16 W [K, N] = fp16_rn(float(s[g(k), n]) * (q[k, n] - ((zstored[g(k), n] + 1) & 15)))."""
    q = unpack_rows(qweight)
    z = (unpack_cols(qzeros) + 1) & 0xF
    K = q.shape[0]
    if g_idx is None:
        gs = K if groupsize == -1 else groupsize
        g = torch.arange(K, dtype=torch.int64) // gs
    else:
        g = g_idx.to(torch.int64)
    return (scales[g].float() * (q - z[g]).float()).half()


def dequant_awq(qweight, qzeros, scales, groupsize=128) -> torch.Tensor:
    """AWQ GEMM layout, zero points used as stored."""
    q = awq_unpack_cols(qweight)
    z = awq_unpack_cols(qzeros)
    K = q.shape[0]
    gs = K if groupsize == -1 else groupsize
    g = torch.arange(K, dtype=torch.int64) // gs
    return (scales[g].float() * (q - z[g]).float()).half()


def linear_forward(x: torch.Tensor, w: torch.Tensor, bias=None):
    """(fp32 result before the cast, fp16 output): x.float() @ W.float(), cast, then the bias in
    fp16 arithmetic (`out + self.bias` on a half tensor, triton.py:351-363)."""
    y32 = x.float() @ w.float()
    y = y32.half()
    if bias is not None:
        y = y + bias
    return y32, y
