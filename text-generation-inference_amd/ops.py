"""Tensor-level wrappers over the C ABI: pointers, shapes, stream and workspace.

PyTorch is used for device memory and streams only; all arithmetic happens in the HIP
kernels of libq4linear.so.  CPU tensors are rejected: there is no host fallback.
"""

from __future__ import annotations

import ctypes
import weakref
from dataclasses import dataclass, field
from typing import Optional

import torch

from . import _lib
from ._lib import (
    DTYPE_BF16,
    DTYPE_F16,
    LAYOUT_AWQ,
    LAYOUT_GPTQ,
    PATH_AUTO,
    Q4Weight,
)

_DTYPES = {torch.float16: DTYPE_F16, torch.bfloat16: DTYPE_BF16}

# (device index, stream handle) -> zero-initialised workspace tensor (uint8)
_workspaces: dict[tuple[int, int], torch.Tensor] = {}
# Workspaces that were replaced by larger ones.  A HIP graph captured earlier holds the raw
# address of the buffer it was recorded with and writes tickets, cells and partial sums there on
# every replay: handing that memory back to the allocator would let replays corrupt whatever
# tensor gets it next.  Buffers grow geometrically, so everything retired stays below the size of
# the live one.
_retired_workspaces: list[torch.Tensor] = []
# weights whose layers were built on the GPU (prepare()), for the load-time tuning pass
_prepared: list = []
# what the last autotune() call measured and chose
last_autotune_report: dict = {}

# row counts whose launch plans a layer fetches when it is built: every decode batch up to 16
# rows and a ladder up to the prefill limit
_PLAN_ROWS = tuple(range(1, 17)) + (17, 20, 24, 32, 33, 48, 64, 65, 96, 128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096)


def _require_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}: the int4 linear kernels run on the GPU only "
            "(no CPU fallback exists in this package)"
        )


def _dense16(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and on a 16-byte boundary (the kernels fetch with 16-byte loads): a view that
    starts elsewhere in its storage is copied."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


@dataclass
class PackedWeight:
    """Validated view of one quantized weight, ready to be passed through the C ABI."""

    qweight: torch.Tensor
    qzeros: torch.Tensor
    scales: torch.Tensor
    g_idx: Optional[torch.Tensor]
    K: int
    N: int
    groupsize: int
    num_groups: int
    layout: int
    # Rows in group order (make_sequential): packed row i holds checkpoint row perm[i] and the
    # kernels take the activation columns in that order; None for checkpoint order.
    perm: Optional[torch.Tensor] = None
    # (M, dtype code) -> (kernel path, workspace bytes): a pure function of the weight's geometry,
    # asked of the library once and kept (one library call per forward afterwards)
    _plans: dict = field(default_factory=dict, repr=False, compare=False)
    _struct: Optional[Q4Weight] = field(default=None, repr=False, compare=False)

    def __deepcopy__(self, memo):
        import copy

        # the cached ctypes struct holds device addresses: a copy gets its own, on first use
        return PackedWeight(
            copy.deepcopy(self.qweight, memo), copy.deepcopy(self.qzeros, memo), copy.deepcopy(self.scales, memo),
            copy.deepcopy(self.g_idx, memo), self.K, self.N, self.groupsize, self.num_groups, self.layout,
            copy.deepcopy(self.perm, memo), dict(self._plans), None)

    def struct(self) -> Q4Weight:
        if self._struct is None:
            self._struct = self._make_struct()
        return self._struct

    def plan(self, M: int, dtype_code: int) -> tuple:
        """(Q4_PATH_* the library picks, workspace bytes the call needs, explicit decode
        configuration or None) for M rows.  The configuration is None until a tuning pass
        (autotune) has measured a faster one than the library's own choice."""
        key = (M, dtype_code)
        got = self._plans.get(key)
        if got is None:
            lib = _lib.load()
            path, need = ctypes.c_int(0), ctypes.c_size_t(0)
            _lib.check(lib.q4_linear_plan(ctypes.byref(self.struct()), M, dtype_code, ctypes.byref(path), ctypes.byref(need)))
            nbytes = int(need.value)
            if self.perm is not None:
                # weight in group order: x is gathered into the tail of the workspace (all but the
                # shortest decode calls, which gather inside the kernel)
                nbytes = max(nbytes, int(lib.q4_workspace_bytes_perm(M, self.K, self.N)))
            got = (int(path.value), nbytes, None)
            self._plans[key] = got
        return got

    def prepare(self, rows=None, max_rows: int = 4096) -> None:
        """Load-time step of a layer: fetch the launch plans of the decode row counts and of a
        ladder of prefill row counts up to `max_rows` (the reference sizes its scratch for
        max_total_tokens at Warmup, layers/gptq/exllamav2.py:159-175), and reserve the device's
        shared workspace for the largest of them, so that a first forward at any of these row
        counts neither asks the library for a plan nor allocates (it can be captured into a HIP
        graph)."""
        if not self.qweight.is_cuda:
            return
        if rows is None:
            rows = tuple(M for M in _PLAN_ROWS if M <= max(max_rows, 16))
            if max_rows > 16 and max_rows not in rows:
                rows = rows + (max_rows,)
        need = max(self.plan(M, DTYPE_F16)[1] for M in rows)
        for M in rows:
            need = max(need, self.plan(M, DTYPE_BF16)[1])
        with torch.cuda.device(self.qweight.device):
            reserve_workspace(self.qweight.device, need, SHARED)
        if not any(r() is self for r in _prepared):
            _prepared.append(weakref.ref(self))

    def _make_struct(self) -> Q4Weight:
        return Q4Weight(
            self.qweight.data_ptr(),
            self.qzeros.data_ptr(),
            self.scales.data_ptr(),
            self.g_idx.data_ptr() if self.g_idx is not None else None,
            self.K,
            self.N,
            self.groupsize,
            self.num_groups,
            self.layout,
        )


def make_packed(qweight, qzeros, scales, g_idx, groupsize: int, layout: int) -> PackedWeight:
    """Check dtypes/shapes the way the reference's extension does before building a matrix.

    Mirrors the TORCH_CHECKs of server/exllamav2_kernels/exllamav2_kernels/ext.cpp:60-70
    (qweight.size(1) == qzeros.size(1) * 8 == scales.size(1), int32 packed tensors).
    """
    for name, t in (("qweight", qweight), ("qzeros", qzeros)):
        if t.dtype != torch.int32:
            raise TypeError(f"{name} must be int32, got {t.dtype}")
    if scales.dtype != torch.float16:
        raise TypeError(f"scales must be float16, got {scales.dtype}")
    if qweight.dim() != 2 or qzeros.dim() != 2 or scales.dim() != 2:
        raise ValueError("qweight, qzeros and scales must be 2-D")
    if layout == LAYOUT_GPTQ:
        K, N = qweight.shape[0] * 8, qweight.shape[1]
    else:
        K, N = qweight.shape[0], qweight.shape[1] * 8
    G = scales.shape[0]
    if scales.shape[1] != N or tuple(qzeros.shape) != (G, N // 8) or N % 8 != 0:
        raise ValueError(
            f"inconsistent shapes: qweight {tuple(qweight.shape)} qzeros {tuple(qzeros.shape)} "
            f"scales {tuple(scales.shape)}"
        )
    groupsize = int(groupsize)
    if groupsize == -1:
        groupsize = K
    if groupsize < 1:
        raise ValueError(f"bad groupsize {groupsize}")
    if g_idx is not None:
        if layout == LAYOUT_AWQ:
            raise ValueError("g_idx is not defined for the AWQ layout")
        if g_idx.dtype != torch.int32:
            g_idx = g_idx.to(torch.int32)
        if g_idx.numel() != K:
            raise ValueError(f"g_idx has {g_idx.numel()} entries, expected {K}")
        g_idx = _dense16(g_idx)
    elif G * groupsize < K:
        raise ValueError(f"{G} groups of {groupsize} rows do not cover K={K}")
    dev = qweight.device
    for name, t in (("qzeros", qzeros), ("scales", scales), ("g_idx", g_idx)):
        if t is not None and t.device != dev:
            raise ValueError(f"{name} is on {t.device}, qweight on {dev}")
    return PackedWeight(
        _dense16(qweight), _dense16(qzeros), _dense16(scales), g_idx, K, N, groupsize, G, layout
    )


def make_sequential(w: PackedWeight) -> Optional[PackedWeight]:
    """Act-order weight with its rows put into group order, or None when that is not possible.

    What the reference's exllamav2 matrix does at load time (QMatrix::make_sequential,
    exllamav2_kernels/cuda/q_matrix.cu:566-640): perm is the stable argsort of g_idx, packed row
    i of the new qweight is checkpoint row perm[i], and the activations are read through perm.
    The contiguous-group kernels then apply (decode 1.5-2x, prefill 2x faster than the kernels
    that look every weight's group up).  Needs every group to hold exactly `groupsize` rows,
    which a GPTQ act-order g_idx (a permutation of arange(K) // groupsize) does.  The new
    qweight is a second [K/8, N] tensor; the caller drops the old one to keep memory flat.
    Runs once per layer at load time (one device->host sync for the check).
    """
    if w.g_idx is None or w.layout != LAYOUT_GPTQ or w.perm is not None:
        return None
    _require_cuda(w.qweight, "qweight")
    K = w.K
    if K % 8 or w.num_groups * w.groupsize != K:
        return None
    g = w.g_idx.to(torch.int64)
    perm = torch.argsort(g, stable=True)
    expect = torch.arange(K, device=g.device, dtype=torch.int64) // w.groupsize
    if not bool(torch.equal(g[perm], expect)):
        return None
    perm32 = perm.to(torch.int32).contiguous()
    out = torch.empty_like(w.qweight)
    with torch.cuda.device(w.qweight.device):
        _lib.check(_lib.load().q4_gptq_make_sequential(
            w.qweight.data_ptr(), perm32.data_ptr(), out.data_ptr(), K, w.N, _stream_handle(out.device)))
    return PackedWeight(out, w.qzeros, w.scales, None, K, w.N, w.groupsize, w.num_groups, w.layout, perm32)


def permute_output_columns(w: PackedWeight, cols: torch.Tensor) -> PackedWeight:
    """The same weight with its output columns reordered: column j of the result is column
    cols[j] of w (GPTQ layout; load-time integer reshuffles, nothing is requantized)."""
    from .layers.awq.conversion_utils import pack, unpack

    if w.layout != LAYOUT_GPTQ:
        raise ValueError("permute_output_columns handles the GPTQ layout")
    cols = cols.to(torch.int64)
    if cols.numel() != w.N:
        raise ValueError(f"cols has {cols.numel()} entries, expected {w.N}")
    qweight = w.qweight.index_select(1, cols).contiguous()
    scales = w.scales.index_select(1, cols).contiguous()
    qzeros = pack(unpack(w.qzeros, "column").index_select(1, cols), "column").contiguous()
    return PackedWeight(qweight, qzeros, scales, w.g_idx, w.K, w.N, w.groupsize, w.num_groups, w.layout, w.perm)


def gather_columns(x: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
    """x[:, perm] for a contiguous fp16/bf16 [M, K] tensor, through the HIP gather kernel."""
    out = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().q4_gather_columns(
                x.data_ptr(), perm.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], _stream_handle(x.device)))
    return out


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_handle(device: torch.device) -> int:
    """The current HIP stream of `device` as an integer handle."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)  # one C call; Stream objects cost about 1 us more
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    """Stand-in for torch.cuda.device(...) when the device is already current."""

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(device: torch.device):
    """Context that makes `device` current for the launches inside it; entering and leaving
    torch.cuda.device costs about 2 us per call, so nothing is switched when it already is."""
    if device.index is None or torch.cuda.current_device() == device.index:
        return _NO_SWITCH
    return torch.cuda.device(device)


# stream key of a device's shared workspace (reserved at load time, used under graph capture)
SHARED = -1


def reserve_workspace(device: torch.device, nbytes: int, stream: Optional[int] = None) -> torch.Tensor:
    """Return this (device, stream)'s workspace, growing it to at least `nbytes`.

    The first bytes hold the split-K ticket counters: they must start at zero and the
    kernels leave them at zero, so a grown buffer is freshly zeroed; the old one is kept (not
    freed), because HIP graphs captured earlier hold its address.
    `stream=SHARED` names the device's shared workspace: the layers reserve it when they are
    built, and calls made while a stream is capturing (where nothing may be allocated or
    cleared) fall back to it.
    """
    if stream is None:
        stream = _stream_handle(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            # a captured graph may still write into the old buffer on replay: it is kept alive,
            # and the new one is at least twice its size so that the retired ones stay bounded
            _retired_workspaces.append(ws)
            nbytes = max(int(nbytes), 2 * ws.numel())
        ws = torch.zeros(int(nbytes), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _workspace_for_call(device: torch.device, need: int, stream: int) -> torch.Tensor:
    """The workspace a kernel call on `stream` uses.  Outside graph capture: the stream's own,
    grown on demand.  Under capture nothing is allocated: the stream's own if it is large
    enough, else the device's shared workspace (calls that share it must be ordered, which the
    nodes of one captured stream are)."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _workspaces.get(key)
    if ws is not None and ws.numel() >= need:
        return ws
    if torch.cuda.is_current_stream_capturing():
        shared = _workspaces.get((key[0], SHARED))
        if shared is not None and (ws is None or shared.numel() > ws.numel()):
            ws = shared
        if ws is None:
            raise RuntimeError(
                "no workspace was reserved before the stream began capturing: build the layer on the GPU "
                "(its post_init reserves one) or call ops.reserve_workspace(device, nbytes, ops.SHARED) first")
        return ws  # a decode call that needs more reports it; a prefill call runs unsplit
    return reserve_workspace(device, need, stream)


def workspace_bytes(M: int, K: int, N: int) -> int:
    return int(_lib.load().q4_workspace_bytes(int(M), int(K), int(N)))


def dequantize(w: PackedWeight, dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """Dense W [K, N] in `dtype`, produced by the HIP dequant kernel."""
    _require_cuda(w.qweight, "qweight")
    if dtype not in _DTYPES:
        raise TypeError(f"dequantize supports float16/bfloat16, got {dtype}")
    out = torch.empty((w.K, w.N), dtype=dtype, device=w.qweight.device)
    with torch.cuda.device(w.qweight.device):
        st = w.struct()
        _lib.check(
            _lib.load().q4_dequant(ctypes.byref(st), out.data_ptr(), _DTYPES[dtype], _stream_handle(out.device))
        )
    if w.perm is not None:  # rows are in group order: hand them back in checkpoint order
        ordered = torch.empty_like(out)
        ordered.index_copy_(0, w.perm.to(torch.int64), out)
        return ordered
    return out


def linear(
    w: PackedWeight,
    x: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    path: int = PATH_AUTO,
    gemv_config: Optional[tuple] = None,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """y[M, N] = x[M, K] @ dequant(W) (+ bias) on the current stream of x's device.

    `out`, if given, must be a contiguous [M, N] tensor of x's dtype on x's device; it is
    written in place (no allocation happens in the call, which keeps it graph-capturable
    with a pre-reserved workspace).
    """
    _require_cuda(x, "x")
    _require_cuda(w.qweight, "qweight")
    if x.device != w.qweight.device:
        raise RuntimeError(f"x is on {x.device}, weights on {w.qweight.device}")
    if x.dtype not in _DTYPES:
        raise TypeError(f"x must be float16 or bfloat16, got {x.dtype}")
    if x.dim() != 2 or x.shape[1] != w.K:
        raise ValueError(f"x must be [M, {w.K}], got {tuple(x.shape)}")
    x = _dense16(x)
    if w.perm is not None and gemv_config is not None:
        x = gather_columns(x, w.perm)  # explicit decode configurations take x in row order
    M = x.shape[0]
    if out is not None:
        if tuple(out.shape) != (M, w.N) or out.dtype != x.dtype or out.device != x.device or not out.is_contiguous():
            raise ValueError(f"out must be a contiguous [{M}, {w.N}] {x.dtype} tensor on {x.device}")
        y = out
    else:
        y = torch.empty((M, w.N), dtype=x.dtype, device=x.device)
    if M == 0 or w.N == 0:
        return y
    fused_bias = bias is not None and bias.dtype == x.dtype and bias.is_cuda and bias.numel() == w.N
    bias_ptr = bias.contiguous().data_ptr() if fused_bias else None
    lib = _lib.load()
    with _on_device(x.device):
        stream = _stream_handle(x.device)
        # decode: split-K partial sums, tickets, accumulation cells; prefill GEMM: split-K
        # partial tiles when the tile grid alone would leave CUs idle
        planned_path, need, tuned = w.plan(M, _DTYPES[x.dtype])
        if path == PATH_AUTO and gemv_config is None:
            path = planned_path
            if tuned is not None and w.perm is None:
                gemv_config = tuned  # the decomposition a tuning pass measured fastest
        ws = _workspace_for_call(x.device, need, stream)
        st = w.struct()
        if gemv_config is not None:
            wcol, wk, splits = gemv_config[:3]
            words = gemv_config[3] if len(gemv_config) > 3 else 4
            need = _lib.WORKSPACE_COUNTER_BYTES + splits * M * w.N * 4
            if ws.numel() < need:
                ws = _workspace_for_call(x.device, need, stream)
            rc = lib.q4_gemv_tuned(
                ctypes.byref(st), x.data_ptr(), bias_ptr, y.data_ptr(), M, _DTYPES[x.dtype],
                ws.data_ptr(), ws.numel(), wcol, wk, splits, words, stream,
            )
        elif w.perm is not None:
            rc = lib.q4_linear_perm(
                ctypes.byref(st), w.perm.data_ptr(), x.data_ptr(), bias_ptr, y.data_ptr(), M, _DTYPES[x.dtype],
                ws.data_ptr(), ws.numel(), path, stream,
            )
        else:
            rc = lib.q4_linear_ex(
                ctypes.byref(st), x.data_ptr(), bias_ptr, y.data_ptr(), M, _DTYPES[x.dtype],
                ws.data_ptr(), ws.numel(), path, stream,
            )
        _lib.check(rc)
    if bias is not None and not fused_bias:
        if out is not None:
            y.add_(bias)
        else:
            y = y + bias
    return y


def _time_graph_launches(fns, reps: int) -> float:
    """Seconds per launch: `reps` launches (rotating over fns) captured into one HIP graph on a
    side stream, replayed and bracketed by events on that stream."""
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fns[0]()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(reps):
                fns[i % len(fns)]()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            graph.replay()
            e1.record(side)
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / reps
            best = t if best is None or t < best else best
    del graph
    return best


def decode_candidates(w: PackedWeight, M: int, dtype: torch.dtype = torch.float16) -> list:
    """Explicit decode configurations the library offers for timing against its own choice."""
    buf = (ctypes.c_int32 * (4 * 64))()
    n = int(_lib.load().q4_gemv_candidates(ctypes.byref(w.struct()), int(M), _DTYPES[dtype], buf, 64))
    _lib.check(n)
    return [tuple(int(buf[4 * i + k]) for k in range(4)) for i in range(n)]


def autotune(weights=None, rows=(1, 2, 3, 4, 8, 16), dtype: torch.dtype = torch.float16, reps: int = 24,
             min_gain: float = 0.03) -> dict:
    """Measured launch plans for the decode row counts, the load-time counterpart of the
    autotuner of the reference's Triton path (layers/gptq/custom_autotune.py:1-80).

    Weights of the same geometry (the layers of one model that share a shape) form a group.  For
    every group and row count the library's own choice and each configuration it offers
    (q4_gemv_candidates) are timed as HIP graphs of `reps` launches that rotate over the group's
    weights (so that a group larger than the last-level cache streams from HBM, as in serving),
    and the fastest one is kept in every weight's plan when it beats the library's choice by
    `min_gain` or more.  `weights=None`: every weight whose layer was built on the GPU.
    Synchronizes the device; call it once after the model is loaded and before any stream
    capture (the layers do: `create_exllama_buffers`, the reference's Warmup hook).
    Returns {(K, N, groupsize, M): (chosen configuration or None, us of the library's choice,
    us of the chosen one)}."""
    if weights is None:
        weights = [r() for r in _prepared]
        weights = [w for w in weights if w is not None]
    groups: dict = {}
    for w in weights:
        if not w.qweight.is_cuda or w.perm is not None:
            continue
        key = (w.qweight.device, w.K, w.N, w.groupsize, w.num_groups, w.layout, w.g_idx is not None)
        groups.setdefault(key, []).append(w)
    code = _DTYPES[dtype]
    report = {}
    lib = _lib.load()
    for (device, K, N, groupsize, _, _, _), ws in groups.items():
        with torch.cuda.device(device):
            rot = ws[:: max(1, len(ws) // 8)][:8]  # up to eight weights of the group, spread over it
            for M in rows:
                if ws[0].plan(M, code)[0] != _lib.PATH_GEMV:
                    continue
                cands = decode_candidates(ws[0], M, dtype)
                if not cands:
                    continue
                x = torch.randn((M, K), device=device, dtype=dtype)
                y = torch.empty((M, N), device=device, dtype=dtype)
                need = max([ws[0].plan(M, code)[1]] + [
                    int(lib.q4_gemv_tuned_workspace_bytes(ctypes.byref(ws[0].struct()), M, code, *cfg)) for cfg in cands])
                reserve_workspace(device, need, SHARED)
                base = _time_graph_launches([(lambda w=w: linear(w, x, None, path=_lib.PATH_GEMV, out=y)) for w in rot], reps)
                best_t, best_cfg = base, None
                for cfg in cands:
                    try:
                        linear(rot[0], x, None, gemv_config=cfg, out=y)  # a decomposition that does not fit (LDS) is skipped
                    except _lib.Q4Error:
                        continue
                    t = _time_graph_launches([(lambda w=w, cfg=cfg: linear(w, x, None, gemv_config=cfg, out=y)) for w in rot], reps)
                    if t < best_t:
                        best_t, best_cfg = t, cfg
                if best_cfg is not None and best_t > (1.0 - min_gain) * base:
                    best_t, best_cfg = base, None
                for w in ws:
                    path, nbytes, _ = w.plan(M, code)
                    w._plans[(M, code)] = (path, max(nbytes, need), best_cfg)
                report[(K, N, groupsize, M)] = (best_cfg, round(base * 1e6, 2), round(best_t * 1e6, 2))
    global last_autotune_report
    last_autotune_report = report
    return report


def act_mul(gate_up: torch.Tensor, act: str = "silu", out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """act(gate_up[:, :I]) * gate_up[:, I:] for a contiguous [M, 2I] fp16/bf16 tensor."""
    _require_cuda(gate_up, "gate_up")
    if gate_up.dtype not in _DTYPES:
        raise TypeError(f"gate_up must be float16 or bfloat16, got {gate_up.dtype}")
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise ValueError(f"gate_up must be [M, 2I], got {tuple(gate_up.shape)}")
    if act not in _lib.ACTIVATIONS:
        raise ValueError(f"unknown activation {act!r}; known: {sorted(_lib.ACTIVATIONS)}")
    gate_up = _dense16(gate_up)
    M, inter = gate_up.shape[0], gate_up.shape[1] // 2
    y = out if out is not None else torch.empty((M, inter), dtype=gate_up.dtype, device=gate_up.device)
    if tuple(y.shape) != (M, inter) or y.dtype != gate_up.dtype or not y.is_contiguous():
        raise ValueError(f"out must be a contiguous [{M}, {inter}] {gate_up.dtype} tensor")
    with torch.cuda.device(gate_up.device):
        _lib.check(_lib.load().q4_act_mul(gate_up.data_ptr(), y.data_ptr(), M, inter, _DTYPES[gate_up.dtype],
                                          _lib.ACTIVATIONS[act], _stream_handle(gate_up.device)))
    return y


def _gate_up_fused_preferred(w: PackedWeight, M: int, dtype_code: int) -> bool:
    """The library's own answer (q4_linear_gate_up_plan) to: one fused launch, or the linear
    kernel followed by the elementwise kernel?  Kept with the weight's plans."""
    key = ("gate_up", M, dtype_code)
    got = w._plans.get(key)
    if got is None:
        fused = ctypes.c_int(0)
        _lib.check(_lib.load().q4_linear_gate_up_plan(ctypes.byref(w.struct()), int(M), dtype_code, ctypes.byref(fused)))
        got = bool(fused.value)
        w._plans[key] = got
    return got


def linear_gate_up(
    w: PackedWeight,
    x: torch.Tensor,
    act: str = "silu",
    bias: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    fused: Optional[bool] = None,
) -> torch.Tensor:
    """y[M, N/2] = act(x @ W[:, :N/2]) * (x @ W[:, N/2:]) for a weight that packs [gate | up].

    One launch where a fused kernel covers the weight (GPTQ layout with contiguous groups);
    otherwise the linear kernel followed by the elementwise act_mul kernel.  `fused`
    forces one of the two (True raises if there is no fused kernel).
    """
    _require_cuda(x, "x")
    _require_cuda(w.qweight, "qweight")
    if x.dtype not in _DTYPES:
        raise TypeError(f"x must be float16 or bfloat16, got {x.dtype}")
    if x.dim() != 2 or x.shape[1] != w.K:
        raise ValueError(f"x must be [M, {w.K}], got {tuple(x.shape)}")
    if w.N % 2:
        raise ValueError(f"N={w.N} cannot hold a gate and an up half")
    if act not in _lib.ACTIVATIONS:
        raise ValueError(f"unknown activation {act!r}; known: {sorted(_lib.ACTIVATIONS)}")
    x = _dense16(x)
    M, inter = x.shape[0], w.N // 2
    y = out if out is not None else torch.empty((M, inter), dtype=x.dtype, device=x.device)
    if tuple(y.shape) != (M, inter) or y.dtype != x.dtype or y.device != x.device or not y.is_contiguous():
        raise ValueError(f"out must be a contiguous [{M}, {inter}] {x.dtype} tensor on {x.device}")
    if M == 0 or inter == 0:
        return y
    fusable_bias = bias is None or (bias.dtype == x.dtype and bias.is_cuda and bias.numel() == w.N)
    if fused is None and not _gate_up_fused_preferred(w, M, _DTYPES[x.dtype]):
        fused = False  # no fused kernel here, or the two launches measured faster (the library's rule)
    if fused is not False and fusable_bias:
        lib = _lib.load()
        with _on_device(x.device):
            stream = _stream_handle(x.device)
            ws = _workspace_for_call(x.device, w.plan(M, _DTYPES[x.dtype])[1], stream)
            st = w.struct()
            rc = lib.q4_linear_gate_up_perm(
                ctypes.byref(st), w.perm.data_ptr() if w.perm is not None else None, x.data_ptr(),
                bias.contiguous().data_ptr() if bias is not None else None,
                y.data_ptr(), M, _DTYPES[x.dtype], _lib.ACTIVATIONS[act], ws.data_ptr(), ws.numel(), stream,
            )
        if rc != _lib.ERR_UNSUPPORTED or fused:
            _lib.check(rc)
            return y
    elif fused:
        raise ValueError("the fused kernel needs a bias of x's dtype with N entries (or none)")
    return act_mul(linear(w, x, bias), act, out=y)


def select_path(w: PackedWeight, M: int, dtype: torch.dtype = torch.float16) -> str:
    st = w.struct()
    rc = _lib.load().q4_select_path(ctypes.byref(st), int(M), _DTYPES[dtype])
    _lib.check(rc)
    return _lib.PATH_NAMES[rc]


# --------------------------------------------------------------------------- mixture of experts


@dataclass
class PackedMoeWeight:
    """The experts of one projection, stacked along a leading expert dimension in checkpoint
    layout: GPTQ qweight [E, K/8, N] (AWQ [E, K, N/8]), qzeros [E, G, N/8], scales [E, G, N],
    optional g_idx [E, K] (GPTQ act-order)."""

    qweight: torch.Tensor
    qzeros: torch.Tensor
    scales: torch.Tensor
    g_idx: Optional[torch.Tensor]
    K: int
    N: int
    groupsize: int
    num_groups: int
    num_experts: int
    layout: int
    # Every expert's rows in group order (make_sequential_moe): perm [E, K] int32, packed row i of
    # expert e holds its checkpoint row perm[e, i]; None for checkpoint order.
    perm: Optional[torch.Tensor] = None

    def struct(self) -> _lib.Q4MoeWeight:
        e0 = _lib.Q4Weight(
            self.qweight.data_ptr(), self.qzeros.data_ptr(), self.scales.data_ptr(),
            self.g_idx.data_ptr() if self.g_idx is not None else None,
            self.K, self.N, self.groupsize, self.num_groups, self.layout,
        )
        return _lib.Q4MoeWeight(
            e0, self.num_experts, self.qweight.stride(0), self.qzeros.stride(0), self.scales.stride(0),
            self.g_idx.stride(0) if self.g_idx is not None else 0,
        )


def make_packed_moe(qweight, qzeros, scales, groupsize: int, g_idx=None, layout: int = LAYOUT_GPTQ) -> PackedMoeWeight:
    """Validate stacked expert tensors and wrap them for the grouped kernels."""
    if qweight.dim() != 3 or qzeros.dim() != 3 or scales.dim() != 3:
        raise ValueError("stacked expert tensors must be [E, ...] with three dimensions")
    E = qweight.shape[0]
    if g_idx is not None and (g_idx.dim() != 2 or g_idx.shape[0] != E):
        raise ValueError(f"g_idx must be [{E}, K], got {tuple(g_idx.shape)}")
    one = make_packed(qweight[0], qzeros[0], scales[0], g_idx[0] if g_idx is not None else None, groupsize, layout)
    if qzeros.shape[0] != E or scales.shape[0] != E:
        raise ValueError(f"expert counts differ: {E}, {qzeros.shape[0]}, {scales.shape[0]}")
    if g_idx is not None:
        g_idx = g_idx.to(torch.int32).contiguous()
    for name, t in (("qweight", qweight), ("qzeros", qzeros), ("scales", scales)):
        if not t[0].is_contiguous():
            raise ValueError(f"{name}: every expert's slice must be contiguous")
    return PackedMoeWeight(qweight, qzeros, scales, g_idx, one.K, one.N, one.groupsize, one.num_groups, E, layout)


def make_sequential_moe(w: PackedMoeWeight) -> Optional[PackedMoeWeight]:
    """Stacked act-order experts with every expert's rows put into group order (see
    make_sequential), or None when some expert's groups are not all `groupsize` rows.
    The new qweight is a second [E, K/8, N] tensor; the caller drops the old one."""
    if w.g_idx is None or w.layout != LAYOUT_GPTQ or w.perm is not None:
        return None
    _require_cuda(w.qweight, "qweight")
    K, E = w.K, w.num_experts
    if K % 8 or w.num_groups * w.groupsize != K:
        return None
    g = w.g_idx.to(torch.int64)
    perm = torch.argsort(g, dim=1, stable=True)
    expect = (torch.arange(K, device=g.device, dtype=torch.int64) // w.groupsize).expand(E, K)
    if not bool(torch.equal(torch.gather(g, 1, perm), expect)):
        return None
    perm32 = perm.to(torch.int32).contiguous()
    out = torch.empty_like(w.qweight)
    lib = _lib.load()
    with torch.cuda.device(w.qweight.device):
        stream = _stream_handle(out.device)
        for e in range(E):
            _lib.check(lib.q4_gptq_make_sequential(
                w.qweight[e].data_ptr(), perm32[e].data_ptr(), out[e].data_ptr(), K, w.N, stream))
    return PackedMoeWeight(out, w.qzeros, w.scales, None, K, w.N, w.groupsize, w.num_groups, E, w.layout, perm32)


def fold_moe_down_permutation(gate_up: PackedMoeWeight, down: PackedMoeWeight):
    """Experts whose down projection is in group order: apply every expert's permutation to the
    output columns of its gate and up halves instead (load time; see permute_output_columns), so
    that the second projection needs no activation gather.  Returns (gate_up, down), unchanged
    when there is nothing to fold."""
    if down.perm is None or gate_up.layout != LAYOUT_GPTQ or gate_up.N != 2 * down.K \
            or gate_up.num_experts != down.num_experts:
        return gate_up, down
    inter = down.K
    parts = []
    for e in range(gate_up.num_experts):
        one = PackedWeight(gate_up.qweight[e], gate_up.qzeros[e], gate_up.scales[e], None, gate_up.K, gate_up.N,
                           gate_up.groupsize, gate_up.num_groups, gate_up.layout)
        perm = down.perm[e].to(torch.int64)
        parts.append(permute_output_columns(one, torch.cat([perm, perm + inter])))
    new_gate_up = PackedMoeWeight(
        torch.stack([p.qweight for p in parts]), torch.stack([p.qzeros for p in parts]),
        torch.stack([p.scales for p in parts]), gate_up.g_idx, gate_up.K, gate_up.N, gate_up.groupsize,
        gate_up.num_groups, gate_up.num_experts, gate_up.layout, gate_up.perm)
    new_down = PackedMoeWeight(down.qweight, down.qzeros, down.scales, None, down.K, down.N, down.groupsize,
                               down.num_groups, down.num_experts, down.layout, None)
    return new_gate_up, new_down


def _moe_gather(w: PackedMoeWeight, x: torch.Tensor, routing: "MoeRouting", gather: bool) -> torch.Tensor:
    """Activations of every sorted row in its expert's row order: [tokens*k, K]."""
    T, k = routing.topk_ids.shape
    out = torch.empty((T * k, w.K), dtype=x.dtype, device=x.device)
    if out.numel():
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().q4_moe_gather_columns(
                x.data_ptr(), routing.sorted_tokens.data_ptr() if gather else None, routing.expert_offsets.data_ptr(),
                w.perm.data_ptr(), out.data_ptr(), w.num_experts, T * k, w.K, _stream_handle(x.device)))
    return out


@dataclass
class MoeRouting:
    """Result of `moe_route`; every tensor lives on the device."""

    topk_weights: torch.Tensor   # f32 [T, k]
    topk_ids: torch.Tensor       # i32 [T, k]
    sorted_tokens: torch.Tensor  # i32 [T*k]: token of every row of the expert-sorted order
    pair_slot: torch.Tensor      # i32 [T*k]: sorted row of pair (t, j)
    expert_offsets: torch.Tensor  # i32 [E+1]


_GATING_DTYPES = {torch.float16: DTYPE_F16, torch.bfloat16: DTYPE_BF16, torch.float32: _lib.DTYPE_F32}


def moe_route(gating_output: torch.Tensor, topk: int, renormalize: bool = True,
              num_expert_group: int = 0, topk_group: int = 0) -> MoeRouting:
    """softmax -> top-k (-> renormalise) per token and the sort of the pairs by expert.
    num_expert_group > 0: grouped top-k (experts are chosen inside the topk_group best groups)."""
    _require_cuda(gating_output, "gating_output")
    if gating_output.dim() != 2 or gating_output.dtype not in _GATING_DTYPES:
        raise ValueError("gating_output must be a [tokens, experts] float16/bfloat16/float32 tensor")
    g = gating_output.contiguous()
    T, E = g.shape
    dev = g.device
    r = MoeRouting(
        torch.empty((T, topk), dtype=torch.float32, device=dev),
        torch.empty((T, topk), dtype=torch.int32, device=dev),
        torch.empty((T * topk,), dtype=torch.int32, device=dev),
        torch.empty((T * topk,), dtype=torch.int32, device=dev),
        torch.empty((E + 1,), dtype=torch.int32, device=dev),
    )
    with torch.cuda.device(dev):
        _lib.check(_lib.load().q4_moe_route_grouped(
            g.data_ptr(), _GATING_DTYPES[g.dtype], T, E, int(topk), int(bool(renormalize)),
            int(num_expert_group or 0), int(topk_group or 0), r.topk_weights.data_ptr(), r.topk_ids.data_ptr(), r.sorted_tokens.data_ptr(), r.pair_slot.data_ptr(),
            r.expert_offsets.data_ptr(), _stream_handle(dev),
        ))
    return r


def moe_linear(w: PackedMoeWeight, x: torch.Tensor, routing: MoeRouting, gather: bool) -> torch.Tensor:
    """Grouped linear layer: sorted row r becomes x_row(r) @ W[expert of r].

    gather=True: x is [tokens, K] and row r reads its token's row (first projection);
    gather=False: x is [tokens*k, K] already in sorted order (second projection).
    Returns y [tokens*k, N] in sorted order.
    """
    _require_cuda(x, "x")
    if x.dtype not in _DTYPES:
        raise TypeError(f"x must be float16 or bfloat16, got {x.dtype}")
    T, k = routing.topk_ids.shape
    rows = T if gather else T * k
    if x.dim() != 2 or tuple(x.shape) != (rows, w.K):
        raise ValueError(f"x must be [{rows}, {w.K}], got {tuple(x.shape)}")
    x = _dense16(x)
    if w.perm is not None and T > 0:
        x = _moe_gather(w, x, routing, gather)  # sorted rows, columns in each expert's row order
        gather = False
    y = torch.empty((T * k, w.N), dtype=x.dtype, device=x.device)
    if T == 0:
        return y
    lib = _lib.load()
    with torch.cuda.device(x.device):
        stream = _stream_handle(x.device)
        st = w.struct()
        ws = reserve_workspace(x.device, int(lib.q4_moe_workspace_bytes(ctypes.byref(st), T, k)), stream)
        _lib.check(lib.q4_moe_linear(
            ctypes.byref(st), x.data_ptr(), routing.sorted_tokens.data_ptr() if gather else None,
            routing.expert_offsets.data_ptr(), y.data_ptr(), T, k, _DTYPES[x.dtype], ws.data_ptr(), ws.numel(), stream,
        ))
    return y


def moe_linear_gate_up(w: PackedMoeWeight, x: torch.Tensor, routing: MoeRouting, act: str = "silu") -> torch.Tensor:
    """First projection of the experts with the gated-MLP tail: sorted row r becomes
    act(x[token(r)] @ gate_e) * (x[token(r)] @ up_e), [tokens*k, N/2].  One fused launch where
    the decode kernel offers it (one token), else grouped linear + act_mul."""
    _require_cuda(x, "x")
    if x.dtype not in _DTYPES:
        raise TypeError(f"x must be float16 or bfloat16, got {x.dtype}")
    if act not in _lib.ACTIVATIONS:
        raise ValueError(f"unknown activation {act!r}; known: {sorted(_lib.ACTIVATIONS)}")
    T, k = routing.topk_ids.shape
    if x.dim() != 2 or tuple(x.shape) != (T, w.K):
        raise ValueError(f"x must be [{T}, {w.K}], got {tuple(x.shape)}")
    x = _dense16(x)
    x_rows = routing.sorted_tokens
    if w.perm is not None and T > 0:
        # experts in group order: sorted rows with their expert's column order, then as below
        x = _moe_gather(w, x, routing, True)
        x_rows = None
        w = PackedMoeWeight(w.qweight, w.qzeros, w.scales, None, w.K, w.N, w.groupsize, w.num_groups,
                            w.num_experts, w.layout)
    if T > 0:
        lib = _lib.load()
        y = torch.empty((T * k, w.N // 2), dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            stream = _stream_handle(x.device)
            st = w.struct()
            ws = reserve_workspace(x.device, int(lib.q4_moe_workspace_bytes(ctypes.byref(st), T, k)), stream)
            rc = lib.q4_moe_linear_gate_up(
                ctypes.byref(st), x.data_ptr(), x_rows.data_ptr() if x_rows is not None else None,
                routing.expert_offsets.data_ptr(),
                y.data_ptr(), T, k, _DTYPES[x.dtype], _lib.ACTIVATIONS[act], ws.data_ptr(), ws.numel(), stream,
            )
        if rc != _lib.ERR_UNSUPPORTED:
            _lib.check(rc)
            return y
    return act_mul(moe_linear(w, x, routing, gather=x_rows is not None), act)


def moe_combine(y_sorted: torch.Tensor, routing: MoeRouting) -> torch.Tensor:
    """out[t] = sum_j topk_weights[t, j] * y_sorted[slot(t, j)] (fp32 sum, one rounding)."""
    _require_cuda(y_sorted, "y_sorted")
    T, k = routing.topk_ids.shape
    y_sorted = y_sorted.contiguous()
    N = y_sorted.shape[1]
    out = torch.empty((T, N), dtype=y_sorted.dtype, device=y_sorted.device)
    if T == 0:
        return out
    with torch.cuda.device(y_sorted.device):
        _lib.check(_lib.load().q4_moe_combine(
            y_sorted.data_ptr(), routing.topk_weights.data_ptr(), routing.pair_slot.data_ptr(), out.data_ptr(),
            T, k, N, _DTYPES[y_sorted.dtype], _stream_handle(y_sorted.device),
        ))
    return out


def moe_forward(gate_up: PackedMoeWeight, down: PackedMoeWeight, x: torch.Tensor, gating_output: torch.Tensor,
                topk: int, renormalize: bool = True, act: str = "silu",
                num_expert_group: int = 0, topk_group: int = 0) -> torch.Tensor:
    """The sparse MoE block: route, [gate | up] projection, act(gate) * up, down projection,
    weighted sum over the chosen experts."""
    routing = moe_route(gating_output, topk, renormalize, num_expert_group, topk_group)
    h = moe_linear_gate_up(gate_up, x, routing, act)
    return moe_combine(moe_linear(down, h, routing, gather=False), routing)
