"""CPU oracle for the int4 weight-only quantized linear layer (GPTQ / AWQ).

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it, and only as the checker.  The product
path (the HIP kernels behind the C-ABI library) never routes through this file.

It restates, in NumPy, the arithmetic the reference performs on this path.  Each
function cites the reference file:line it follows (paths relative to the reference
checkout root).

Pinning status (what proves each function right, other than itself):
  unpack_rows / unpack_cols / pack_rows / pack_cols
        pinned: literal known-answer words (0x76543210 etc.), round trips through an
        independent restatement of the reference's writer (QuantLinear.pack), pure
        Python element-wise brute force on tiny shapes.
  gptq_zero_points (+1 rule)
        pinned: the reference writer stores z-1 (triton.py:326) so writer->reader round
        trip recovers W only with the +1; literal 0x77777777 -> 8.
  awq_unpack_cols / awq_pack_cols / fast_awq_to_gptq
        pinned: ORDER/REVERSE are mutual inverses, literal words, and the equivalence
        dequant_awq(q, z, s) == dequant_gptq(*fast_awq_to_gptq(q, z), s) bit for bit.
  dequant_gptq / dequant_awq
        pinned: closed-form cases (constant nibbles), writer round trip, g_idx
        permutation invariance, trivial g_idx == no g_idx, IEEE single-rounding check
        against float64.
  matmul_fp32 / linear_forward
        pinned: float64 matmul, linearity, identity/one-hot activations that read
        single weight rows back.
  moe_fused_topk
        pinned: scipy.special.softmax + argsort brute force, hand-computed two-expert case,
        weights sum to 1 after renormalisation; follows the in-tree pure-PyTorch routine.
  moe_grouped_topk
        pinned: brute force from the definition (group maxima, kept groups, masked top-k) and
        the special cases one group (== moe_fused_topk) and all groups kept (== moe_fused_topk).
  moe_forward
        structure pinned by the in-tree dense formulation it follows (every expert applied
        to every token, weighted by the scattered top-k weights) through its already pinned
        parts (linear_forward, gate_up_forward).  The reference's GPTQ MoE kernels
        (kernels-community/moe, fused_marlin_moe) are not in the tree: their internal
        roundings are parity unpinned; GPU results are compared within the GEMM tolerance.
  gptq_find_params / gptq_fasterquant (the solver, float64)
        pinned: with a diagonal Hessian the result is round-to-nearest with the group ranges
        (closed form); for any Hessian dW H dW^T / 2 equals the returned error exactly (the
        algebra of the Cholesky update: it caught a transposed factor); every value sits on its
        group's 16-level grid; the output error on correlated inputs is below round-to-nearest's;
        dead inputs give zero columns and act_order walks the columns by decreasing activity.
        The reference runs these loops in fp32 on the GPU: its decisions near rounding ties
        are not pinned bit for bit (GPU agreement is asserted for >= 97 % of the nibbles).
  awq_inference_engine.gemm_forward_cuda (third-party, huggingface/llm-awq @ bd1dc2d5,
  not in the reference tree): parity unpinned by any runnable reference test; covered
  through the in-tree equivalence fast_awq_to_gptq (awq/conversion_utils.py:83-97).
"""

from __future__ import annotations

import numpy as np

# server/text_generation_server/layers/awq/conversion_utils.py:5-6
AWQ_PACK_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]
REVERSE_AWQ_PACK_ORDER = [0, 4, 1, 5, 2, 6, 3, 7]

_SHIFTS = np.arange(0, 32, 4, dtype=np.uint32)


def _as_u32(a: np.ndarray) -> np.ndarray:
    a = np.asarray(a)
    if a.dtype == np.int32:
        return a.view(np.uint32)
    if a.dtype == np.uint32:
        return a
    raise TypeError(f"packed tensors must be int32/uint32, got {a.dtype}")


# --------------------------------------------------------------------------- unpack / pack


def unpack_rows(qmatrix: np.ndarray) -> np.ndarray:
    """[R, C] packed words -> [8R, C] nibbles; nibble j of word [r, c] is element [8r+j, c].

    Follows layers/gptq/triton.py:160-169,191 (shifter = (k % 8) * 4 on qweight rows) and
    layers/awq/conversion_utils.py:52-55 (direction="row").
    """
    q = _as_u32(qmatrix)
    out = (q[:, None, :] >> _SHIFTS[None, :, None]) & np.uint32(0xF)
    return out.reshape(q.shape[0] * 8, q.shape[1]).astype(np.uint8)


def unpack_cols(qmatrix: np.ndarray) -> np.ndarray:
    """[R, C] packed words -> [R, 8C] nibbles; nibble j of word [r, c] is element [r, 8c+j].

    Follows layers/gptq/triton.py:167,170,184 (zeros_shifter = (n % 8) * 4),
    exllamav2_kernels/cuda/matrix_view.cuh:85-119 and conversion_utils.py:47-50.
    """
    q = _as_u32(qmatrix)
    out = (q[:, :, None] >> _SHIFTS[None, None, :]) & np.uint32(0xF)
    return out.reshape(q.shape[0], q.shape[1] * 8).astype(np.uint8)


def pack_rows(imatrix: np.ndarray) -> np.ndarray:
    """Inverse of unpack_rows (conversion_utils.py:26-28; writer triton.py:316-324)."""
    i = (np.asarray(imatrix).astype(np.int64) & 0xF).astype(np.uint32)
    assert i.shape[0] % 8 == 0
    i = i.reshape(i.shape[0] // 8, 8, i.shape[1])
    q = np.bitwise_or.reduce(i << _SHIFTS[None, :, None], axis=1)
    return q.astype(np.uint32).view(np.int32)


def pack_cols(imatrix: np.ndarray) -> np.ndarray:
    """Inverse of unpack_cols (conversion_utils.py:22-24; writer triton.py:332-343)."""
    i = (np.asarray(imatrix).astype(np.int64) & 0xF).astype(np.uint32)
    assert i.shape[1] % 8 == 0
    i = i.reshape(i.shape[0], i.shape[1] // 8, 8)
    q = np.bitwise_or.reduce(i << _SHIFTS[None, None, :], axis=2)
    return q.astype(np.uint32).view(np.int32)


def awq_unpack_cols(qmatrix: np.ndarray) -> np.ndarray:
    """AWQ GEMM layout -> logical [R, 8C] nibbles.

    Position p of word [r, c] holds logical column 8c + AWQ_PACK_ORDER[p]
    (conversion_utils.py:83-92: unpack by columns then reorder with REVERSE_AWQ_PACK_ORDER).
    """
    raw = unpack_cols(qmatrix)
    r = raw.reshape(raw.shape[0], -1, 8)[:, :, REVERSE_AWQ_PACK_ORDER]
    return r.reshape(raw.shape)


def awq_pack_cols(imatrix: np.ndarray) -> np.ndarray:
    """Logical [R, 8C] nibbles -> AWQ GEMM layout words (inverse of awq_unpack_cols)."""
    i = np.asarray(imatrix)
    r = i.reshape(i.shape[0], -1, 8)[:, :, AWQ_PACK_ORDER].reshape(i.shape)
    return pack_cols(r)


def fast_awq_to_gptq(qweight: np.ndarray, qzeros: np.ndarray):
    """AWQ (qweight [K, N/8], qzeros [G, N/8]) -> GPTQ (qweight [K/8, N], qzeros [G, N/8]).

    Follows conversion_utils.py:83-97: un-interleave, subtract 1 from the zero points
    (masked to 4 bits by pack), repack weights by rows and zeros by columns.
    """
    izeros = awq_unpack_cols(qzeros).astype(np.int16) - 1
    iweights = awq_unpack_cols(qweight)
    return pack_rows(iweights), pack_cols(izeros)


# --------------------------------------------------------------------------- dequant


def gptq_zero_points(qzeros: np.ndarray) -> np.ndarray:
    """[G, N/8] words -> effective zero points [G, N] = (stored + 1) & 0xF.

    Follows triton.py:184-185, exllamav2 q_gemm_kernel_gptq.cuh:155-158,
    exllama q4_matmul.cu:89 and gaudi hpu.py:58-69 (all apply the same +1).
    """
    return ((unpack_cols(qzeros).astype(np.int16) + 1) & 0xF).astype(np.uint8)


def group_index(K: int, groupsize: int, g_idx: np.ndarray | None) -> np.ndarray:
    """Group of every input row: g_idx[k] if given, else k // groupsize (triton.py:174-182)."""
    if g_idx is not None:
        g = np.asarray(g_idx).astype(np.int64)
        assert g.shape == (K,)
        return g
    if groupsize == -1:
        groupsize = K
    return np.arange(K, dtype=np.int64) // groupsize


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even, NaN kept quiet."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    nan = np.isnan(a)
    rounded = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded)
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def _scale_diff(scales: np.ndarray, q: np.ndarray, z: np.ndarray, g: np.ndarray, dtype: str):
    """W[k, n] = round_dtype(float(s[g(k), n]) * float(q[k, n] - z[g(k), n])).

    The product of an 11-bit significand and an integer of magnitude <= 15 is exact in
    float32, so rounding it once to fp16 equals the reference's single fp16 multiply
    (triton.py:192; q_matrix.cu:282-293; q4_matrix.cu:194-202).  For bf16 the same exact
    product is rounded once to bf16 (extension; the reference is fp16-only here).
    """
    s = np.asarray(scales)
    assert s.dtype == np.float16, "scales are fp16 on this path (gptq/__init__.py:29-31)"
    diff = q.astype(np.int16) - z[g].astype(np.int16)
    prod = s[g].astype(np.float32) * diff.astype(np.float32)
    if dtype == "f16":
        return prod.astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(prod)
    raise ValueError(dtype)


def dequant_gptq(qweight, qzeros, scales, g_idx=None, groupsize=128, dtype="f16"):
    """Dense W [K, N] (np.float16, or uint16 bf16 bit patterns) from GPTQ tensors.

    Follows triton.py:139-192 (layout + arithmetic) and gaudi hpu.py:58-78.
    """
    q = unpack_rows(qweight)
    z = gptq_zero_points(qzeros)
    K, N = q.shape
    assert z.shape[1] == N and scales.shape == z.shape, (q.shape, z.shape, scales.shape)
    g = group_index(K, groupsize, g_idx)
    assert g.min() >= 0 and g.max() < z.shape[0]
    return _scale_diff(scales, q, z, g, dtype)


def dequant_awq(qweight, qzeros, scales, groupsize=128, dtype="f16"):
    """Dense W [K, N] from AWQ GEMM-layout tensors; zero points are used as stored.

    Follows awq/conversion_utils.py:35-97 (layout) and gaudi awq/quantize/hpu.py:22-72
    (W = s * (q - z), no +1).
    """
    q = awq_unpack_cols(qweight)
    z = awq_unpack_cols(qzeros)
    K, N = q.shape
    assert z.shape[1] == N and scales.shape == z.shape, (q.shape, z.shape, scales.shape)
    g = group_index(K, groupsize, None)
    assert g.max() < z.shape[0]
    return _scale_diff(scales, q, z, g, dtype)


# --------------------------------------------------------------------------- matmul / forward


def to_f32(a: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "f16":
        assert a.dtype == np.float16
        return a.astype(np.float32)
    if dtype == "bf16":
        assert a.dtype == np.uint16
        return bf16_bits_to_f32(a)
    raise ValueError(dtype)


def matmul_fp32(x_f32: np.ndarray, w_f32: np.ndarray) -> np.ndarray:
    """y = x @ W with float32 accumulation (the fp32-accumulated reference of the parity bar)."""
    return np.matmul(x_f32.astype(np.float32), w_f32.astype(np.float32))


def linear_forward(x, w, bias=None, dtype="f16"):
    """Reference forward contract (triton.py:351-363; awq/quantize/cuda.py:43-49).

    x: [..., K] in `dtype`; w: dense dequantized [K, N] in `dtype`.  Returns
    (y_f32 [..., N] before the output cast, y_cast in `dtype`).  The bias is added after
    the matmul result has been cast to the activation dtype, as the reference does
    (`out + self.bias` on an fp16 tensor).
    """
    K, N = w.shape
    lead = x.shape[:-1]
    x2 = to_f32(x.reshape(-1, K), dtype)
    y = matmul_fp32(x2, to_f32(w, dtype))
    if dtype == "f16":
        yc = y.astype(np.float16)
        if bias is not None:
            yc = (yc.astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
            y = y + bias.astype(np.float32)
    else:
        yc = f32_to_bf16_bits(y)
        if bias is not None:
            yc = f32_to_bf16_bits(bf16_bits_to_f32(yc) + bf16_bits_to_f32(bias))
            y = y + bf16_bits_to_f32(bias)
    return y.reshape(lead + (N,)), yc.reshape(lead + (N,))


def activation_f32(g: np.ndarray, act: str) -> np.ndarray:
    """The reference's MLP activations in fp32 (ACT2FN / torch.nn.functional.gelu selection,
    server/text_generation_server/models/custom_modeling/flash_llama_modeling.py:309-321):
    "silu" = g * sigmoid(g); "gelu_tanh" = gelu(approximate="tanh"); "gelu" = erf form."""
    g = g.astype(np.float32)
    if act == "silu":
        return (g / (np.float32(1.0) + np.exp(-g, dtype=np.float32))).astype(np.float32)
    if act == "gelu_tanh":
        inner = np.float32(0.7978845608028654) * (g + np.float32(0.044715) * g * g * g)
        return (np.float32(0.5) * g * (np.float32(1.0) + np.tanh(inner, dtype=np.float32))).astype(np.float32)
    if act == "gelu":
        from math import erf

        e = np.vectorize(erf, otypes=[np.float64])(g.astype(np.float64) * 0.7071067811865476)
        return (0.5 * g.astype(np.float64) * (1.0 + e)).astype(np.float32)
    raise ValueError(f"unknown activation {act}")


def gate_up_forward(x, w, act="silu", bias=None, dtype="f16"):
    """act(gate) * up of a gated MLP whose first linear packs [gate | up] along N
    (flash_llama_modeling.py:400-404), with eager PyTorch's roundings on half tensors:
    the linear output is rounded to `dtype`, the activation is evaluated in fp32 and
    rounded, the product is rounded.  Returns (y_f32 from the unrounded fp32 linear output,
    y_cast in `dtype`); both [..., N/2]."""
    y32, yc = linear_forward(x, w, bias, dtype)
    inter = w.shape[1] // 2
    exact = activation_f32(y32[..., :inter], act) * y32[..., inter:]
    yr = to_f32(yc, dtype)
    a = activation_f32(yr[..., :inter], act)
    if dtype == "f16":
        a = a.astype(np.float16).astype(np.float32)
        out = (a * yr[..., inter:]).astype(np.float16)
    else:
        a = bf16_bits_to_f32(f32_to_bf16_bits(a))
        out = f32_to_bf16_bits(a * yr[..., inter:])
    return exact, out


# --------------------------------------------------------------------------- mixture of experts


def moe_fused_topk(gating: np.ndarray, topk: int, renormalize: bool):
    """Routing of the sparse MoE layers (server/text_generation_server/layers/moe/
    fused_moe_ipex.py:53-65): softmax over the experts in fp32, the `topk` largest
    probabilities per token (descending; equal values: lowest expert first), optionally
    renormalised to sum 1.  Returns (weights f32 [T, topk], ids int32 [T, topk])."""
    g = np.asarray(gating).astype(np.float32)
    e = np.exp(g - g.max(axis=1, keepdims=True), dtype=np.float32)
    prob = (e / e.sum(axis=1, keepdims=True, dtype=np.float32)).astype(np.float32)
    ids = np.argsort(-prob, axis=1, kind="stable")[:, :topk]
    w = np.take_along_axis(prob, ids, axis=1)
    if renormalize:
        w = w / w.sum(axis=1, keepdims=True, dtype=np.float32)
    return w.astype(np.float32), ids.astype(np.int32)


def moe_grouped_topk(gating: np.ndarray, topk: int, renormalize: bool, num_expert_group: int, topk_group: int):
    """Grouped routing (layers/moe/fused_moe_ipex.py:21-50): softmax over all experts, the
    score of a group is its largest member, the `topk_group` best groups stay, every expert
    outside them is masked to 0, then top-k and the optional renormalisation as above."""
    g = np.asarray(gating).astype(np.float32)
    T, E = g.shape
    e = np.exp(g - g.max(axis=1, keepdims=True), dtype=np.float32)
    prob = (e / e.sum(axis=1, keepdims=True, dtype=np.float32)).astype(np.float32)
    group_scores = prob.reshape(T, num_expert_group, -1).max(axis=2)
    keep = np.argsort(-group_scores, axis=1, kind="stable")[:, :topk_group]
    mask = np.zeros((T, num_expert_group), dtype=bool)
    np.put_along_axis(mask, keep, True, axis=1)
    masked = np.where(np.repeat(mask, E // num_expert_group, axis=1), prob, np.float32(0.0))
    ids = np.argsort(-masked, axis=1, kind="stable")[:, :topk]
    w = np.take_along_axis(masked, ids, axis=1)
    if renormalize:
        w = w / w.sum(axis=1, keepdims=True, dtype=np.float32)
    return w.astype(np.float32), ids.astype(np.int32)


def moe_forward(x, gating, gate_up_w, down_w, topk, renormalize=True, act="silu", dtype="f16"):
    """Sparse MoE block, following the reference's dense formulation
    (layers/moe/__init__.py:158-194): out = sum_e weights[:, e] * down_e(act(gate_e(x)) * up_e(x))
    with weights the top-k routing weights scattered over the experts (zero elsewhere, so
    only chosen experts are evaluated here).  gate_up_w[e] is the dense [K, 2I] weight that
    packs [gate | up], down_w[e] the dense [I, K] one.  Every expert's projections carry the
    roundings of linear_forward / gate_up_forward; the weighted sum is kept in fp32 and
    rounded once.  Returns (out_f32, out_cast)."""
    T = x.shape[0]
    w, ids = moe_fused_topk(gating, topk, renormalize)
    H = down_w[0].shape[1]
    out = np.zeros((T, H), dtype=np.float32)
    for e in sorted(set(ids.reshape(-1).tolist())):
        rows, slots = np.nonzero(ids == e)
        _, h = gate_up_forward(x[rows], gate_up_w[e], act, None, dtype)
        _, d = linear_forward(h, down_w[e], None, dtype)
        out[rows] += w[rows, slots][:, None] * to_f32(d, dtype)
    cast = out.astype(np.float16) if dtype == "f16" else f32_to_bf16_bits(out)
    return out, cast


# --------------------------------------------------------------------------- synthetic inputs


def _gptq_round(x, scale, zero):
    """Quantizer._quantize (quantize.py:54-58): scale * (clamp(round(x / scale) + zero, 0, 15) - zero)."""
    return scale * (np.clip(np.rint(x / scale) + zero, 0, 15) - zero)


def gptq_find_params(x, sym, mse=False, norm=2.4, grid=100, maxshrink=0.8):
    """Range rule of the reference's quantizer (quantize.py:60-130): per row of x (float64), the
    range always contains 0; sym mirrors it; an all-zero row gets [-1, 1].  With mse the range
    is shrunk by p = 1 - i / grid for i = 0 .. maxshrink * grid - 1 and a row keeps the first
    candidate with the smallest sum of |quantized - x| ** norm (:101-123; sym keeps zero = 8).
    Returns (scale, zero) per row, 4 bits."""
    x = np.asarray(x, dtype=np.float64)
    lo = np.minimum(x.min(axis=1), 0.0)
    hi = np.maximum(x.max(axis=1), 0.0)
    if sym:
        hi = np.maximum(np.abs(lo), hi)
        lo = np.where(lo < 0, -hi, lo)
    dead = (lo == 0) & (hi == 0)
    lo = np.where(dead, -1.0, lo)
    hi = np.where(dead, 1.0, hi)
    scale = (hi - lo) / 15.0
    zero = np.full_like(scale, 8.0) if sym else np.rint(-lo / scale)
    if mse:
        best = np.full(x.shape[0], np.inf)
        zero0 = zero.copy()
        for i in range(int(maxshrink * grid)):
            p = 1 - i / grid
            scale1 = (p * hi - p * lo) / 15.0
            zero1 = zero0 if sym else np.rint(-(p * lo) / scale1)
            err = np.sum(np.abs(_gptq_round(x, scale1[:, None], zero1[:, None]) - x) ** norm, axis=1)
            better = err < best
            best = np.where(better, err, best)
            scale = np.where(better, scale1, scale)
            zero = np.where(better, zero1, zero)
    return scale, zero


def gptq_fasterquant(W, H, blocksize=128, percdamp=0.01, groupsize=-1, act_order=False, sym=True, mse=False):
    """The GPTQ solver in float64, column by column (quantize.py:243-351).

    W [rows, K] (one row per output feature), H [K, K] the accumulated Hessian 2/n X X^T.
    Dead inputs (H_ii = 0) get H_ii = 1 and zero weights; act_order walks the columns by
    decreasing H_ii; H is damped by percdamp * mean(diag); U is the upper Cholesky factor of
    inv(H).  Every column is rounded with its group's (scale, zero) (found when the group starts,
    from the values its columns had when the block started) and its error (w - q) / U_ii is subtracted, times U[i, c],
    from every later column c.  Returns Q (dequantized values, checkpoint column order),
    scale [rows, G], zero [rows, G], g_idx [K], error = sum of (w - q)^2 / U_ii^2 / 2, and the
    damped (and, with act_order, permuted) H together with the column order used.
    Plain loops: for small cases only."""
    W = np.array(W, dtype=np.float64)
    H = np.array(H, dtype=np.float64)
    rows, K = W.shape
    # one group for all of K: the range comes from the weights as given, dead inputs included
    # (quantizer.find_params(W) runs before the dead columns are cleared, quantize.py:257-264)
    whole = gptq_find_params(W, sym, mse) if groupsize == -1 else None
    dead = np.diag(H) == 0
    H[dead, dead] = 1.0
    W[:, dead] = 0.0
    perm = np.arange(K)
    if act_order:
        perm = np.argsort(-np.diag(H), kind="stable")
        W = W[:, perm]
        H = H[perm][:, perm]
    H[np.arange(K), np.arange(K)] += percdamp * np.mean(np.diag(H))
    Hinv = np.linalg.inv(H)
    U = np.linalg.cholesky(Hinv).T  # upper factor: inv(H) = U^T U (torch.linalg.cholesky(upper=True))
    Q = np.zeros_like(W)
    error = 0.0
    gs = K if groupsize == -1 else groupsize
    G = (K + gs - 1) // gs
    scale = np.zeros((rows, G))
    zero = np.zeros((rows, G))
    if groupsize == -1:
        scale[:, 0], zero[:, 0] = whole
    for i1 in range(0, K, blocksize):
        i2 = min(i1 + blocksize, K)
        Err = np.zeros((rows, i2 - i1))
        W1 = W[:, i1:i2].copy()  # the block's working copy; W keeps the values of block entry
        for i in range(i1, i2):
            g = i // gs
            if groupsize != -1 and i % gs == 0:
                # from W, which has the updates of finished blocks only (quantize.py:308-312)
                scale[:, g], zero[:, g] = gptq_find_params(W[:, i:i + gs], sym, mse)
            w = W1[:, i - i1]
            d = U[i, i]
            q = scale[:, g] * (np.clip(np.rint(w / scale[:, g]) + zero[:, g], 0, 15) - zero[:, g])
            Q[:, i] = q
            error += float(np.sum((w - q) ** 2 / d ** 2)) / 2
            err = (w - q) / d
            W1[:, i - i1:] -= np.outer(err, U[i, i:i2])
            Err[:, i - i1] = err
        W[:, i2:] -= Err @ U[i1:i2, i2:]
    g_idx = (np.arange(K) // gs).astype(np.int32)
    Hd = H
    if act_order:
        inv = np.argsort(perm)
        Q = Q[:, inv]
        g_idx = g_idx[inv]
    return Q, scale, zero, g_idx, error, Hd, perm


def make_gptq(K, N, groupsize=128, seed=0, sym=True, act_order=False):
    """Seeded synthetic GPTQ tensors of the benchmark's shape.

    nibbles uniform 0..15 packed 8 per int32 along K; scales fp16 uniform [1e-3, 2e-2];
    sym -> stored zero nibble 7 (effective 8, the value the reference writer emits for
    symmetric quantisation, triton.py:326-343), else uniform 0..15; act_order ->
    g_idx[perm[i]] = i // groupsize for a random permutation (every group has exactly
    `groupsize` rows).
    """
    rng = np.random.default_rng(seed)
    gs = K if groupsize == -1 else groupsize
    G = (K + gs - 1) // gs
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    qweight = pack_rows(q)
    if sym:
        zs = np.full((G, N), 7, dtype=np.uint8)
    else:
        zs = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    qzeros = pack_cols(zs)
    scales = rng.uniform(1e-3, 2e-2, size=(G, N)).astype(np.float16)
    g_idx = None
    if act_order:
        perm = rng.permutation(K)
        g_idx = np.empty(K, dtype=np.int32)
        g_idx[perm] = (np.arange(K) // gs).astype(np.int32)
    return qweight, qzeros, scales, g_idx


def make_awq(K, N, groupsize=128, seed=0):
    """Seeded synthetic AWQ GEMM-layout tensors: nibbles and zero points uniform 0..15."""
    rng = np.random.default_rng(seed)
    gs = K if groupsize == -1 else groupsize
    G = K // gs
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    scales = rng.uniform(1e-3, 2e-2, size=(G, N)).astype(np.float16)
    return awq_pack_cols(q), awq_pack_cols(z), scales


def make_x(M, K, seed=0, dtype="f16"):
    """Activations ~ N(0, 1) in the given dtype (fp16 array, or bf16 bit patterns)."""
    rng = np.random.default_rng(seed + 7919)
    x = rng.standard_normal((M, K), dtype=np.float32)
    return x.astype(np.float16) if dtype == "f16" else f32_to_bf16_bits(x)
