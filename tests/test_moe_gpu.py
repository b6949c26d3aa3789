"""Mixture of experts on the GPU: routing, the grouped linear layer (decode and MFMA
kernels), the weighted sum and the whole block, against the oracle."""

from __future__ import annotations

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from .util import max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu

TOL = 2e-3       # fp16: max |y - ref| / max |ref| against the fp32-accumulated oracle
TOL_BF16 = 8e-3  # bf16 outputs carry 8 mantissa bits


def _gating(rng, T, E, dtype):
    g = (rng.standard_normal((T, E)) * 2).astype(np.float32)
    t = torch.from_numpy(g)
    if dtype == "f16":
        t = t.half()
    elif dtype == "bf16":
        t = t.bfloat16()
    return t, t.float().numpy()


def _check_routing_structure(r, T, E, k):
    ids = r.topk_ids.cpu().numpy()
    off = r.expert_offsets.cpu().numpy()
    tok = r.sorted_tokens.cpu().numpy()
    slot = r.pair_slot.cpu().numpy()
    assert off[0] == 0 and off[E] == T * k and (np.diff(off) >= 0).all()
    assert sorted(slot.tolist()) == list(range(T * k))  # a permutation of the rows
    counts = np.bincount(ids.reshape(-1), minlength=E)
    assert np.array_equal(np.diff(off), counts)
    for p in range(T * k):
        t, j = divmod(p, k)
        s = slot[p]
        assert tok[s] == t
        e = ids[t, j]
        assert off[e] <= s < off[e + 1]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (5, 8, 2), (16, 8, 1), (300, 64, 6), (4096, 8, 2), (3, 256, 8)])
def test_route(pkg, oracle, gpu, T, E, k, dtype):
    rng = np.random.default_rng(T + E + k)
    g, g32 = _gating(rng, T, E, dtype)
    for renorm in (True, False):
        r = pkg.ops.moe_route(g.to(gpu), k, renorm)
        torch.cuda.synchronize()
        w, ids = oracle.moe_fused_topk(g32, k, renorm)
        assert np.array_equal(r.topk_ids.cpu().numpy(), ids)
        assert np.allclose(r.topk_weights.cpu().numpy(), w, rtol=1e-5, atol=1e-7)
        _check_routing_structure(r, T, E, k)


@pytest.mark.parametrize("T,E,groups,keep,k", [(1, 16, 4, 2, 3), (33, 160, 8, 3, 6), (300, 64, 8, 4, 8), (7, 8, 8, 2, 2),
                                              (5, 12, 3, 1, 4), (4, 64, 32, 5, 5)])
def test_route_grouped(pkg, oracle, gpu, T, E, groups, keep, k):
    rng = np.random.default_rng(T + E)
    g, g32 = _gating(rng, T, E, "f32")
    for renorm in (True, False):
        r = pkg.ops.moe_route(g.to(gpu), k, renorm, groups, keep)
        w, ids = oracle.moe_grouped_topk(g32, k, renorm, groups, keep)
        assert np.array_equal(r.topk_ids.cpu().numpy(), ids)
        assert np.allclose(r.topk_weights.cpu().numpy(), w, rtol=1e-5, atol=1e-7)
        _check_routing_structure(r, T, E, k)


def test_route_grouped_rejects_bad_groups(pkg, gpu):
    z = torch.zeros((2, 16), device=gpu)
    for groups, keep, k in ((3, 1, 2), (4, 5, 2), (4, 1, 5), (64, 2, 2)):
        with pytest.raises(pkg._lib.Q4Error):
            pkg.ops.moe_route(z, k, True, groups, keep)


def test_route_ties_take_the_lowest_expert(pkg, gpu):
    r = pkg.ops.moe_route(torch.zeros((2, 8), device=gpu), 2, True)
    assert r.topk_ids.cpu().tolist() == [[0, 1], [0, 1]]
    assert np.allclose(r.topk_weights.cpu().numpy(), 0.5)


def test_route_rejects_bad_arguments(pkg, gpu):
    with pytest.raises(pkg._lib.Q4Error):
        pkg.ops.moe_route(torch.zeros((2, 8), device=gpu), 9, True)      # topk > experts
    with pytest.raises(pkg._lib.Q4Error):
        pkg.ops.moe_route(torch.zeros((2, 300), device=gpu), 2, True)    # too many experts


def _experts(oracle, gpu, E, K, N, gs, dtype, seed, sym=False):
    """Stacked device tensors and the dense dequantized matrices of E experts."""
    qws, qzs, scs, dense = [], [], [], []
    for e in range(E):
        qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=seed + e, sym=sym)
        qws.append(qw); qzs.append(qz); scs.append(sc)
        dense.append(oracle.dequant_gptq(qw, qz, sc, None, gs, dtype))
    stack = lambda a: to_dev(np.stack(a), gpu)
    return stack(qws), stack(qzs), stack(scs), dense


def _packed_experts(pkg, oracle, gpu, kind, E, K, N, gs, dtype, seed):
    """PackedMoeWeight + dense matrices for kind in {"gptq", "act", "awq"}."""
    qws, qzs, scs, gis, dense = [], [], [], [], []
    for e in range(E):
        if kind == "awq":
            qw, qz, sc = oracle.make_awq(K, N, gs, seed=seed + e)
            dense.append(oracle.dequant_awq(qw, qz, sc, gs, dtype))
        else:
            qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=seed + e, sym=False, act_order=(kind == "act"))
            dense.append(oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype))
            if gi is not None:
                gis.append(gi)
        qws.append(qw); qzs.append(qz); scs.append(sc)
    stack = lambda a: to_dev(np.stack(a), gpu)
    w = pkg.ops.make_packed_moe(stack(qws), stack(qzs), stack(scs), gs, stack(gis) if gis else None,
                                1 if kind == "awq" else 0)
    return w, dense


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("T,E,k,K,N,gs", [
    (1, 8, 2, 1024, 512, 128),      # decode, most experts without rows
    (4, 8, 2, 1024, 512, 128),
    (16, 8, 2, 2048, 1024, 128),    # decode, 16 rows possible per expert
    (7, 4, 4, 1024, 256, 64),       # every token on every expert
    (3, 8, 2, 43 * 128, 256, 128),  # 43 chunks of 128 rows: uneven K ranges
    (5, 8, 2, 512, 256, 32),
    (3, 8, 2, 1024, 512, -1),       # one group
    (17, 8, 2, 1024, 512, 128),
    (40, 2, 2, 1024, 512, 128),     # decode kernel, 40 rows per expert: three row blocks each
    (64, 8, 2, 2048, 512, 128),     # last size of the decode kernel
    (65, 8, 2, 1024, 512, 128),     # first size of the MFMA kernel (split-K: few tiles)
    (100, 8, 2, 4096, 256, 128),    # MFMA kernel, deeper split-K
    (200, 8, 2, 1024, 768, 128),    # 128-column tiles (N not a multiple of 256)
    (300, 4, 1, 512, 512, 64),
    (130, 8, 2, 512, 256, 32),
])
def test_moe_linear_gather(pkg, oracle, gpu, T, E, k, K, N, gs, dtype):
    """First projection: sorted row r = x[token(r)] @ W[expert(r)]."""
    bf = dtype == "bf16"
    rng = np.random.default_rng(T * 7 + E + K)
    qw, qz, sc, dense = _experts(oracle, gpu, E, K, N, gs, dtype, seed=T + K)
    w = pkg.ops.make_packed_moe(qw, qz, sc, gs)
    g, g32 = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = oracle.make_x(T, K, seed=T, dtype=dtype)
    y = pkg.ops.moe_linear(w, to_dev(x, gpu, bf16=bf), r, gather=True)
    torch.cuda.synchronize()
    y = to_f32(y)
    assert np.isfinite(y).all()
    ids = r.topk_ids.cpu().numpy()
    slot = r.pair_slot.cpu().numpy()
    ref = np.zeros_like(y)
    for e in range(E):
        rows, js = np.nonzero(ids == e)
        if rows.size:
            y32, _ = oracle.linear_forward(x[rows], dense[e], None, dtype)
            ref[slot[rows * k + js]] = y32
    err = max_rel_err(y, ref)
    assert err <= (TOL_BF16 if bf else TOL), f"max rel err {err:.3e}"


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("kind", ["act", "awq"])
@pytest.mark.parametrize("T,E,k,K,N,gs", [
    (1, 8, 2, 1024, 512, 128),      # decode kernels (act-order: fp16 only, bf16 takes the MFMA kernel)
    (9, 4, 2, 2048, 512, 128),
    (16, 4, 4, 1024, 256, 64),      # 16 rows on every expert
    (17, 8, 2, 1024, 512, 128),     # MFMA kernel (LDS unpack), split-K
    (150, 4, 2, 1024, 256, 128),    # two row tiles on some experts
    (40, 8, 2, 8192, 128, 32),      # act-order: 256 groups, parameters gathered from global memory
])
def test_moe_linear_act_order_and_awq(pkg, oracle, gpu, kind, T, E, k, K, N, gs, dtype):
    bf = dtype == "bf16"
    rng = np.random.default_rng(T + K + len(kind))
    w, dense = _packed_experts(pkg, oracle, gpu, kind, E, K, N, gs, dtype, seed=T + 3)
    g, _ = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = oracle.make_x(T, K, seed=T, dtype=dtype)
    y = to_f32(pkg.ops.moe_linear(w, to_dev(x, gpu, bf16=bf), r, gather=True))
    assert np.isfinite(y).all()
    ids = r.topk_ids.cpu().numpy()
    slot = r.pair_slot.cpu().numpy()
    ref = np.zeros_like(y)
    for e in range(E):
        rows, js = np.nonzero(ids == e)
        if rows.size:
            ref[slot[rows * k + js]], _ = oracle.linear_forward(x[rows], dense[e], None, dtype)
    err = max_rel_err(y, ref)
    assert err <= (TOL_BF16 if bf else TOL), f"max rel err {err:.3e}"
    # second projection form: x already sorted
    xs = oracle.make_x(T * k, K, seed=T + 1, dtype=dtype)
    y2 = to_f32(pkg.ops.moe_linear(w, to_dev(xs, gpu, bf16=bf), r, gather=False))
    off = r.expert_offsets.cpu().numpy()
    ref2 = np.zeros_like(y2)
    for e in range(E):
        if off[e + 1] > off[e]:
            ref2[off[e]:off[e + 1]], _ = oracle.linear_forward(xs[off[e]:off[e + 1]], dense[e], None, dtype)
    assert max_rel_err(y2, ref2) <= (TOL_BF16 if bf else TOL)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("T,E,k,K,N,gs", [(1, 8, 2, 1024, 512, 128), (9, 4, 2, 2048, 512, 128),
                                          (100, 8, 2, 1024, 256, 64), (16, 4, 4, 43 * 128, 256, 128)])
def test_moe_linear_act_order_rows_in_group_order(pkg, oracle, gpu, T, E, k, K, N, gs, dtype):
    """Act-order experts repacked once (make_sequential_moe): every expert's rows are its
    checkpoint rows in the order of a stable sort of its g_idx, activations are gathered per
    sorted row with the row's expert's permutation, and both projection forms agree with the
    oracle's act-order matrices."""
    bf = dtype == "bf16"
    rng = np.random.default_rng(T + K)
    w, dense = _packed_experts(pkg, oracle, gpu, "act", E, K, N, gs, dtype, seed=T + 5)
    seq = pkg.ops.make_sequential_moe(w)
    assert seq is not None and seq.g_idx is None and tuple(seq.perm.shape) == (E, K)
    perm = seq.perm.cpu().numpy()
    gi = w.g_idx.cpu().numpy()
    for e in range(E):
        assert np.array_equal(gi[e][perm[e]], np.arange(K) // (K if gs == -1 else gs))
        rows = oracle.unpack_rows(w.qweight[e].cpu().numpy())
        assert np.array_equal(oracle.unpack_rows(seq.qweight[e].cpu().numpy()), rows[perm[e]])
    g, _ = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = oracle.make_x(T, K, seed=T, dtype=dtype)
    y = to_f32(pkg.ops.moe_linear(seq, to_dev(x, gpu, bf16=bf), r, gather=True))
    ids = r.topk_ids.cpu().numpy()
    slot = r.pair_slot.cpu().numpy()
    ref = np.zeros_like(y)
    for e in range(E):
        rows, js = np.nonzero(ids == e)
        if rows.size:
            ref[slot[rows * k + js]], _ = oracle.linear_forward(x[rows], dense[e], None, dtype)
    assert max_rel_err(y, ref) <= (TOL_BF16 if bf else TOL)
    xs = oracle.make_x(T * k, K, seed=T + 1, dtype=dtype)
    y2 = to_f32(pkg.ops.moe_linear(seq, to_dev(xs, gpu, bf16=bf), r, gather=False))
    off = r.expert_offsets.cpu().numpy()
    ref2 = np.zeros_like(y2)
    for e in range(E):
        if off[e + 1] > off[e]:
            ref2[off[e]:off[e + 1]], _ = oracle.linear_forward(xs[off[e]:off[e + 1]], dense[e], None, dtype)
    assert max_rel_err(y2, ref2) <= (TOL_BF16 if bf else TOL)
    # the gated first projection takes the two-kernel route on such weights
    if N % 2 == 0:
        xd = to_dev(x, gpu, bf16=bf)
        h = pkg.ops.moe_linear_gate_up(seq, xd, r, "silu")
        assert tuple(h.shape) == (T * k, N // 2)
        two = pkg.ops.act_mul(pkg.ops.moe_linear(seq, xd, r, gather=True), "silu")
        assert max_rel_err(to_f32(h), to_f32(two)) <= (TOL_BF16 if bf else TOL)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("T,E,k,K,I,gs,act", [
    (1, 8, 2, 1024, 512, 128, "silu"),       # fused decode kernel
    (1, 8, 2, 2048, 1024, 128, "gelu_tanh"),
    (1, 4, 4, 43 * 128, 256, 256, "silu"),   # uneven K ranges, every expert chosen
    (2, 8, 2, 2048, 1024, 128, "silu"),      # two tokens: two-kernel route
    (1, 8, 2, 1024, 512, 64, "silu"),        # groups of 64 rows: grouped linear + act_mul
    (3, 8, 2, 1024, 512, 128, "silu"),       # three tokens: two-kernel route
])
def test_moe_linear_gate_up(pkg, oracle, gpu, T, E, k, K, I, gs, act, dtype):
    bf = dtype == "bf16"
    rng = np.random.default_rng(T + K + I)
    qw, qz, sc, dense = _experts(oracle, gpu, E, K, 2 * I, gs, dtype, seed=T + I)
    w = pkg.ops.make_packed_moe(qw, qz, sc, gs)
    g, _ = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = oracle.make_x(T, K, seed=T + 2, dtype=dtype)
    y = pkg.ops.moe_linear_gate_up(w, to_dev(x, gpu, bf16=bf), r, act)
    torch.cuda.synchronize()
    assert y.shape == (T * k, I)
    y = to_f32(y)
    ids = r.topk_ids.cpu().numpy()
    slot = r.pair_slot.cpu().numpy()
    ref = np.zeros_like(y)
    oracle_act = {"gelu_tanh": "gelu_tanh"}.get(act, act)
    for e in range(E):
        rows, js = np.nonzero(ids == e)
        if rows.size:
            ref[slot[rows * k + js]], _ = oracle.gate_up_forward(x[rows], dense[e], oracle_act, None, dtype)
    err = max_rel_err(y, ref)
    assert err <= 2 * (TOL_BF16 if bf else TOL), f"max rel err {err:.3e}"


@pytest.mark.parametrize("T", [2, 16, 40])
def test_moe_linear_sorted_input(pkg, oracle, gpu, T):
    """Second projection: x is already in sorted order."""
    E, k, K, N, gs = 8, 2, 1024, 512, 128
    rng = np.random.default_rng(T)
    qw, qz, sc, dense = _experts(oracle, gpu, E, K, N, gs, "f16", seed=3)
    w = pkg.ops.make_packed_moe(qw, qz, sc, gs)
    g, _ = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = oracle.make_x(T * k, K, seed=T, dtype="f16")
    y = to_f32(pkg.ops.moe_linear(w, to_dev(x, gpu), r, gather=False))
    off = r.expert_offsets.cpu().numpy()
    ref = np.zeros_like(y)
    for e in range(E):
        if off[e + 1] > off[e]:
            ref[off[e]:off[e + 1]], _ = oracle.linear_forward(x[off[e]:off[e + 1]], dense[e], None, "f16")
    assert max_rel_err(y, ref) <= TOL


def test_moe_linear_twice_leaves_the_workspace_clean(pkg, oracle, gpu):
    """The split-K tickets are left at zero: a second call and a plain linear call on the same
    workspace give the same results."""
    E, k, K, N, gs, T = 8, 2, 4096, 1024, 128, 2
    rng = np.random.default_rng(0)
    qw, qz, sc, dense = _experts(oracle, gpu, E, K, N, gs, "f16", seed=50, sym=True)
    w = pkg.ops.make_packed_moe(qw, qz, sc, gs)
    g, _ = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = to_dev(oracle.make_x(T, K, seed=1), gpu)
    a = pkg.ops.moe_linear(w, x, r, gather=True)
    b = pkg.ops.moe_linear(w, x, r, gather=True)
    assert torch.equal(a, b)
    one = pkg.ops.make_packed(qw[0], qz[0], sc[0], None, gs, 0)
    y1 = pkg.ops.linear(one, x)
    y32, _ = oracle.linear_forward(oracle.make_x(T, K, seed=1), dense[0], None, "f16")
    assert max_rel_err(to_f32(y1), y32) <= TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("T,k,N", [(1, 2, 512), (9, 6, 4096), (70000, 1, 8)])
def test_moe_combine(pkg, gpu, T, k, N, dtype):
    rng = np.random.default_rng(T + k)
    td = torch.bfloat16 if dtype == "bf16" else torch.float16
    y = torch.from_numpy(rng.standard_normal((T * k, N)).astype(np.float32)).to(td).to(gpu)
    w = torch.from_numpy(rng.uniform(0.1, 1.0, size=(T, k)).astype(np.float32)).to(gpu)
    slot = torch.from_numpy(rng.permutation(T * k).astype(np.int32)).to(gpu)
    r = pkg.ops.MoeRouting(w, torch.zeros((T, k), dtype=torch.int32, device=gpu), slot, slot, slot[:1])
    out = pkg.ops.moe_combine(y, r)
    ref = (y.float()[slot.long()].reshape(T, k, N) * w[:, :, None]).sum(dim=1)
    assert torch.allclose(out.float(), ref, rtol=1e-2 if dtype == "bf16" else 2e-3, atol=1e-3)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("T,E,k,H,I,gs,act", [
    (1, 8, 2, 1024, 2048, 128, "silu"),
    (6, 8, 2, 1024, 2048, 128, "silu"),
    (16, 4, 2, 512, 1024, 64, "gelu_tanh"),
    (100, 8, 2, 512, 1024, 128, "silu"),
])
def test_moe_block(pkg, oracle, gpu, T, E, k, H, I, gs, act, dtype):
    """route -> [gate | up] -> act(gate) * up -> down -> weighted sum, against the oracle."""
    bf = dtype == "bf16"
    rng = np.random.default_rng(T + H)
    gq, gz, gsc, gu = _experts(oracle, gpu, E, H, 2 * I, gs, dtype, seed=100)
    dq, dz, dsc, dn = _experts(oracle, gpu, E, I, H, gs, dtype, seed=200)
    g, g32 = _gating(rng, T, E, "f32")
    x = oracle.make_x(T, H, seed=T + 1, dtype=dtype)
    ref32, _ = oracle.moe_forward(x, g32, gu, dn, k, True, act, dtype)
    out = pkg.ops.moe_forward(pkg.ops.make_packed_moe(gq, gz, gsc, gs), pkg.ops.make_packed_moe(dq, dz, dsc, gs),
                              to_dev(x, gpu, bf16=bf), g.to(gpu), k, True, act)
    torch.cuda.synchronize()
    assert out.shape == (T, H) and out.dtype == (torch.bfloat16 if bf else torch.float16)
    err = max_rel_err(to_f32(out), ref32)
    # two chained projections with a rounded intermediate: twice the single-GEMM budget
    assert err <= 2 * (TOL_BF16 if bf else TOL), f"max rel err {err:.3e}"


def test_moe_block_mixtral_shape_decode(pkg, oracle, gpu):
    """Mixtral-8x7B expert shapes (hidden 4096, intermediate 14336), two experts, one token."""
    T, E, k, H, I, gs = 1, 2, 2, 4096, 14336, 128
    gq, gz, gsc, gu = _experts(oracle, gpu, E, H, 2 * I, gs, "f16", seed=300, sym=True)
    dq, dz, dsc, dn = _experts(oracle, gpu, E, I, H, gs, "f16", seed=400, sym=True)
    g = torch.tensor([[0.3, -0.2]], dtype=torch.float32)
    x = oracle.make_x(T, H, seed=9)
    ref32, _ = oracle.moe_forward(x, g.numpy(), gu, dn, k, True, "silu", "f16")
    out = pkg.ops.moe_forward(pkg.ops.make_packed_moe(gq, gz, gsc, gs), pkg.ops.make_packed_moe(dq, dz, dsc, gs),
                              to_dev(x, gpu), g.to(gpu), k, True, "silu")
    assert max_rel_err(to_f32(out), ref32) <= 2 * TOL


@pytest.mark.parametrize("desc_act", [False, True])
def test_sparse_moe_layer_from_safetensors(pkg, oracle, gpu, tmp_path, desc_act):
    """The layer class loads per-expert checkpoint tensors through the package's Weights and
    matches the oracle; leading dimensions of x are kept.  desc_act: every projection has a
    permuted g_idx (gate and up of an expert share theirs, as a checkpoint's do)."""
    E, k, H, I, gs = 4, 2, 256, 512, 64
    tensors, gu, dn = {}, [], []
    for e in range(E):
        parts = []
        perm_rng = np.random.default_rng(1000 + e)
        g_in = (np.arange(H) // gs).astype(np.int32)
        g_mid = (np.arange(I) // gs).astype(np.int32)
        if desc_act:
            g_in, g_mid = g_in[perm_rng.permutation(H)], g_mid[perm_rng.permutation(I)]
        for name, (K, N), seed in (("gate_proj", (H, I), 1), ("up_proj", (H, I), 2), ("down_proj", (I, H), 3)):
            qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=10 * e + seed, sym=False)
            gi = g_in if K == H else g_mid
            pre = f"moe.experts.{e}.{name}"
            tensors[f"{pre}.qweight"] = torch.from_numpy(qw.view(np.int32).copy())
            tensors[f"{pre}.qzeros"] = torch.from_numpy(qz.view(np.int32).copy())
            tensors[f"{pre}.scales"] = torch.from_numpy(sc.copy())
            tensors[f"{pre}.g_idx"] = torch.from_numpy(gi.copy())
            parts.append(oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16"))
        gu.append(np.concatenate(parts[:2], axis=1))
        dn.append(parts[2])
    path = tmp_path / "model.safetensors"
    save_file(tensors, str(path))
    from types import SimpleNamespace

    loader = pkg.GPTQWeightsLoader(bits=4, groupsize=gs, desc_act=desc_act, quant_method="gptq", quantize="gptq",
                                   sym=False, modules_to_not_convert=[])
    weights = pkg.Weights([path], gpu, torch.float16, SimpleNamespace(rank=lambda: 0, size=lambda: 1), loader)
    layer = pkg.GPTQSparseMoELayer(n_expert_group=None, n_experts=E, prefix="moe.experts", renormalize=True, topk=k,
                                   topk_group=None, weights=weights)
    import importlib
    mode = importlib.import_module("text-generation-inference_amd.layers.moe").ACT_ORDER_MODE
    if mode == "table":  # checkpoint order kept: the lookup kernels take the stacked g_idx
        assert (layer._gate_up.g_idx is not None) == desc_act and layer._gate_up.perm is None
    else:  # act-order experts are put into group order once: no g_idx left, a permutation per expert
        assert layer._gate_up.g_idx is None and layer._down.g_idx is None
        assert (layer._gate_up.perm is not None) == desc_act
    if desc_act and mode != "table":
        # the down projections' input order went into the gate_up columns: no gather in between
        assert layer._down.perm is None and layer._gate_up.perm is not None
        assert layer.down_proj.rows_in_group_order and layer.down_proj.packed().g_idx is None
    rng = np.random.default_rng(5)
    x = oracle.make_x(6, H, seed=2)
    g = rng.standard_normal((6, E)).astype(np.float32)
    out = layer(to_dev(x, gpu).reshape(2, 3, H), gating_output=torch.from_numpy(g).to(gpu))
    assert out.shape == (2, 3, H)
    ref32, _ = oracle.moe_forward(x, g, gu, dn, k, True, "silu", "f16")
    assert max_rel_err(to_f32(out).reshape(6, H), ref32) <= 2 * TOL


@pytest.mark.parametrize("T", [1, 7, 90])
def test_expert_down_permutations_folded_into_gate_up_columns(pkg, oracle, gpu, T):
    """Folding every expert's down-projection permutation into its gate and up columns leaves the
    block's output bit for bit as with the activation gather between the projections."""
    E, k, H, I, gs = 4, 2, 1024, 512, 128
    gu, _ = _packed_experts(pkg, oracle, gpu, "act", E, H, 2 * I, gs, "f16", seed=3)
    dn, _ = _packed_experts(pkg, oracle, gpu, "act", E, I, H, gs, "f16", seed=9)
    gu, dn = pkg.ops.make_sequential_moe(gu), pkg.ops.make_sequential_moe(dn)
    fgu, fdn = pkg.ops.fold_moe_down_permutation(gu, dn)
    assert fdn.perm is None and fgu.perm is not None
    assert pkg.ops.fold_moe_down_permutation(fgu, fdn)[1] is fdn  # nothing left to fold
    rng = np.random.default_rng(T)
    g, _ = _gating(rng, T, E, "f32")
    x = to_dev(oracle.make_x(T, H, seed=T), gpu)
    want = pkg.ops.moe_forward(gu, dn, x, g.to(gpu), k, True, "silu")
    got = pkg.ops.moe_forward(fgu, fdn, x, g.to(gpu), k, True, "silu")
    assert torch.equal(got, want)


def test_awq_layout_experts_are_converted_once(pkg, oracle, gpu):
    """The layer's weight holder turns AWQ-layout experts into the GPTQ layout when it builds its
    kernel view (same dense matrices bit for bit) and the grouped GPTQ kernels serve them."""
    import importlib
    moe = importlib.import_module("text-generation-inference_amd.layers.moe")
    E, k, K, N, gs, T = 4, 2, 1024, 512, 128, 5
    qws, qzs, scs, dense = [], [], [], []
    for e in range(E):
        qw, qz, sc = oracle.make_awq(K, N, gs, seed=40 + e)
        qws.append(qw); qzs.append(qz); scs.append(sc)
        dense.append(oracle.dequant_awq(qw, qz, sc, gs, "f16"))
    stack = lambda a: to_dev(np.stack(a), gpu)
    holder = moe.GPTQMoEWeight(stack(qws), stack(qzs), stack(scs), None, gs, True)
    if moe.AWQ_MODE == "native":
        pytest.skip("Q4_AWQ=native keeps the AWQ layout")
    w = holder.packed()
    assert w.layout == 0 and tuple(holder.qweight.shape) == (E, K // 8, N) and not holder.use_awq_kernel
    for e in range(E):
        one = pkg.ops.make_packed(holder.qweight[e], holder.qzeros[e], holder.scales[e], None, gs, 0)
        assert np.array_equal(pkg.ops.dequantize(one).cpu().numpy().view(np.uint16), dense[e].view(np.uint16))
    rng = np.random.default_rng(1)
    g, _ = _gating(rng, T, E, "f32")
    r = pkg.ops.moe_route(g.to(gpu), k, True)
    x = oracle.make_x(T, K, seed=3)
    y = to_f32(pkg.ops.moe_linear(w, to_dev(x, gpu), r, gather=True))
    ids = r.topk_ids.cpu().numpy()
    slot = r.pair_slot.cpu().numpy()
    ref = np.zeros_like(y)
    for e in range(E):
        rows, js = np.nonzero(ids == e)
        if rows.size:
            ref[slot[rows * k + js]], _ = oracle.linear_forward(x[rows], dense[e], None, "f16")
    assert max_rel_err(y, ref) <= TOL
