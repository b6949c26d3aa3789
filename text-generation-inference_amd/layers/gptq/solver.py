"""GPTQ: the solver that chooses the 4-bit weights of one linear layer from calibration inputs.

Mirrors the interface of the reference's `GPTQ` class
(server/text_generation_server/layers/gptq/quantize.py:147-375): `add_batch(inp, out)`
accumulates the Hessian 2/n * X X^T of the layer's inputs, `fasterquant(...)` returns
(scale, zero, g_idx, error) and leaves the quantized weights in `layer.weight`, ready for
`QuantLinear.pack`.  The Hessian products, the two Cholesky factorizations and the update of
the columns behind a block are library linear algebra (torch on the GPU, as in the
reference); the column loop inside a block -- 128 dependent steps that the reference runs as
several small kernels each -- is one launch of the HIP kernel behind q4_gptq_solve_block.
Linear layers only (the reference also unfolds Conv2d / transformers.Conv1D inputs).  The
quantizer's range rule runs inside the kernel; with `mse=True` (the reference's grid search over
shrunken ranges, quantize.py:101-123, off by default there too) the ranges of the groups that
start in a block are found with torch before the block's launch and handed to the kernel.
"""

from __future__ import annotations

import math

import torch
import torch.nn as nn

from ... import _lib

BLOCK = 128  # columns per kernel launch


def find_params(x: torch.Tensor, sym: bool, mse: bool = False, norm: float = 2.4, grid: int = 100,
                maxshrink: float = 0.8):
    """Quantizer.find_params for 4 bits, one range per row of x [rows, n] (quantize.py:60-130):
    the range contains 0, sym mirrors it, an all-zero row gets [-1, 1]; with mse the first of the
    ranges shrunk by 1 - i / grid with the smallest sum of |quantized - x| ** norm is kept."""
    zeros = torch.zeros(x.shape[0], device=x.device, dtype=x.dtype)
    lo = torch.minimum(x.min(dim=1).values, zeros)
    hi = torch.maximum(x.max(dim=1).values, zeros)
    return _params_from_range(x, lo, hi, sym, mse, norm, grid, maxshrink)


def _params_from_range(x, lo, hi, sym, mse, norm, grid, maxshrink):
    if sym:
        hi = torch.maximum(lo.abs(), hi)
        lo = torch.where(lo < 0, -hi, lo)
    flat = (lo == 0) & (hi == 0)
    lo = torch.where(flat, torch.full_like(lo, -1), lo)
    hi = torch.where(flat, torch.full_like(hi, 1), hi)
    scale = (hi - lo) / 15
    zero = torch.full_like(scale, 8) if sym else torch.round(-lo / scale)
    if mse:
        best = torch.full_like(scale, float("inf"))
        zero0 = zero.clone()
        for i in range(int(maxshrink * grid)):
            p = 1 - i / grid
            scale1 = (p * hi - p * lo) / 15
            zero1 = zero0 if sym else torch.round(-(p * lo) / scale1)
            q = scale1[:, None] * (torch.clamp(torch.round(x / scale1[:, None]) + zero1[:, None], 0, 15) - zero1[:, None])
            err = (q - x).abs_().pow_(norm).sum(dim=1)
            better = err < best
            best = torch.where(better, err, best)
            scale = torch.where(better, scale1, scale)
            zero = torch.where(better, zero1, zero)
    return scale, zero


class GPTQ:
    def __init__(self, layer: nn.Module, sym: bool = True, mse: bool = False, norm: float = 2.4, grid: int = 100,
                 maxshrink: float = 0.8):
        if not isinstance(layer, nn.Linear):
            raise NotImplementedError("the solver handles nn.Linear layers")
        self.layer = layer
        self.dev = layer.weight.device
        self.rows, self.columns = layer.weight.shape
        self.H = torch.zeros((self.columns, self.columns), device=self.dev, dtype=torch.float32)
        self.nsamples = 0
        self.sym = bool(sym)
        self.mse, self.norm, self.grid, self.maxshrink = bool(mse), float(norm), int(grid), float(maxshrink)

    def add_batch(self, inp: torch.Tensor, out: torch.Tensor = None):
        """H <- running mean of 2 x x^T over all calibration rows (quantize.py:170-216)."""
        if inp.dim() == 2:
            inp = inp.unsqueeze(0)
        batch = inp.shape[0]
        x = inp.reshape(-1, inp.shape[-1]).t().float()  # [columns, tokens]
        self.H *= self.nsamples / (self.nsamples + batch)
        self.nsamples += batch
        x = math.sqrt(2 / self.nsamples) * x
        self.H += x.matmul(x.t())

    @torch.no_grad()
    def fasterquant(self, blocksize: int = BLOCK, percdamp: float = 0.01, groupsize: int = -1,
                    act_order: bool = False, name: str = ""):
        if not self.H.is_cuda:
            raise RuntimeError("the GPTQ solver runs on the GPU only (no CPU fallback exists in this package)")
        if blocksize < 1 or blocksize > BLOCK:
            raise ValueError(f"blocksize must be 1..{BLOCK}, got {blocksize}")
        K, rows = self.columns, self.rows
        W = self.layer.weight.data.clone().float().contiguous()
        # one group for all of K: the row ranges come from the weights as given, before the
        # columns of dead inputs are cleared (quantize.py:257-264)
        whole = None
        if groupsize == -1:
            whole = find_params(W, self.sym, self.mse, self.norm, self.grid, self.maxshrink)
        H = self.H.clone()
        dead = torch.diag(H) == 0
        H[dead, dead] = 1
        W[:, dead] = 0
        perm = None
        if act_order:
            perm = torch.argsort(torch.diag(H), descending=True)
            W = W[:, perm].contiguous()
            H = H[perm][:, perm]
        diag = torch.arange(K, device=self.dev)
        H[diag, diag] += percdamp * torch.mean(torch.diag(H))
        # upper factor U of inv(H): inv(H) = U^T U
        L = torch.linalg.cholesky(H)
        Hinv = torch.cholesky_inverse(L)
        try:
            U = torch.linalg.cholesky(Hinv, upper=True)
        except Exception:  # the reference's fallback for a factorization that fails (quantize.py:282-286)
            U = torch.linalg.cholesky(Hinv + 1e-5 * torch.eye(K, device=self.dev), upper=True)
        U = U.contiguous()

        gs = K if groupsize == -1 else int(groupsize)
        G = (K + gs - 1) // gs
        Q = torch.zeros_like(W)
        scale = torch.zeros((rows, G), device=self.dev, dtype=torch.float32)
        zero = torch.zeros((rows, G), device=self.dev, dtype=torch.float32)
        loss = torch.zeros((rows,), device=self.dev, dtype=torch.float32)
        err = torch.zeros((rows, BLOCK), device=self.dev, dtype=torch.float32)
        if groupsize == -1:
            scale[:, 0], zero[:, 0] = whole
        lib = _lib.load()
        with torch.cuda.device(self.dev):
            stream = torch.cuda.current_stream(self.dev).cuda_stream
            for i1 in range(0, K, blocksize):
                count = min(blocksize, K - i1)
                flags = int(self.sym)
                if self.mse and groupsize != -1:
                    # groups that start in this block: ranges searched on W as it is now (it holds
                    # the updates of finished blocks only, which is what the reference reads)
                    flags |= 2
                    for start in range(-(-i1 // gs) * gs, i1 + count, gs):
                        scale[:, start // gs], zero[:, start // gs] = find_params(
                            W[:, start:start + gs], self.sym, True, self.norm, self.grid, self.maxshrink)
                _lib.check(lib.q4_gptq_solve_block(
                    W.data_ptr(), U.data_ptr(), Q.data_ptr(), err.data_ptr(), loss.data_ptr(), scale.data_ptr(),
                    zero.data_ptr(), rows, K, i1, count, -1 if groupsize == -1 else gs, G, flags, stream))
                i2 = i1 + count
                if i2 < K:
                    W[:, i2:] -= err[:, :count].matmul(U[i1:i2, i2:])
        error = float(loss.sum().item())
        g_idx = (torch.arange(K, device=self.dev) // gs).to(torch.int32)
        if perm is not None:
            invperm = torch.argsort(perm)
            Q = Q[:, invperm]
            g_idx = g_idx[invperm]
        self.layer.weight.data = Q.reshape(self.layer.weight.shape).to(self.layer.weight.data.dtype)
        return scale, zero, g_idx, error

    def free(self):
        self.H = None
        torch.cuda.empty_cache()


@torch.no_grad()
def quantize_linear(layer: nn.Linear, calibration: torch.Tensor, groupsize: int = 128, act_order: bool = False,
                    sym: bool = True, percdamp: float = 0.01, mse: bool = False):
    """Calibrate, solve and pack one linear layer: the per-layer body of the reference's
    `sequential` (layers/gptq/quantize.py:703-735: add_batch over the calibration inputs, fasterquant,
    free) followed by `pack` (:780-791).  `calibration` is [..., in_features] on the layer's (GPU) device; returns
    (QuantLinear on that device, error).  The layer's weight is left holding the quantized values."""
    from .quant_linear import QuantLinear

    solver = GPTQ(layer, sym=sym, mse=mse)
    x = calibration.reshape(-1, calibration.shape[-1])
    for chunk in x.split(4096):  # one "batch" per chunk keeps the Hessian update a bounded GEMM
        solver.add_batch(chunk.unsqueeze(0))
    scale, zero, g_idx, error = solver.fasterquant(percdamp=percdamp, groupsize=groupsize, act_order=act_order)
    solver.free()
    packed = QuantLinear.new(4, groupsize, layer.in_features, layer.out_features, layer.bias is not None)
    packed.pack(layer, scale.cpu(), zero.cpu(), g_idx.cpu())
    return packed.to(layer.weight.device), error
