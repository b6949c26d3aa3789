"""HIP graph capture of the hot path: every replay must reproduce the eager result.

The kernels keep state in the workspace (split-K tickets, accumulation cells, partial sums, the
gathered activations of weights in group order) and promise to leave the counters at zero; a
graph replays the same launches on the same buffers, with eager calls on the same workspace in
between.  All kernels are deterministic, so the comparison is bit for bit."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def to_dev(a, gpu):
    if a is None:
        return None
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


def capture_and_check(torch_fn_list, gpu, between):
    """Eager results, then one graph of all calls replayed three times with eager work between."""
    eager = [fn(None).clone() for fn in torch_fn_list]
    outs = [torch.empty_like(e) for e in eager]
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for fn, o in zip(torch_fn_list, outs):
            fn(o)  # reserves this stream's workspace before capture
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for fn, o in zip(torch_fn_list, outs):
                fn(o)
    torch.cuda.synchronize()
    for replay in range(3):
        for o in outs:
            o.fill_(float("nan"))
        with torch.cuda.stream(side):
            graph.replay()
        torch.cuda.synchronize()
        for i, (o, e) in enumerate(zip(outs, eager)):
            assert torch.equal(o, e), f"replay {replay}, call {i}"
        with torch.cuda.stream(side):
            between()  # eager calls on the same stream and workspace
        torch.cuda.synchronize()


def test_dense_paths_under_graph_replay(pkg, oracle, gpu):
    K, N, gs = 4096, 1024, 128
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=3, sym=False)
    plain = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    aq, agi = oracle.make_gptq(K, N, gs, seed=4, sym=False, act_order=True), None
    act = pkg.ops.make_packed(to_dev(aq[0], gpu), to_dev(aq[1], gpu), to_dev(aq[2], gpu), to_dev(aq[3], gpu), gs, 0)
    seq = pkg.ops.make_sequential(act)
    wq, wz, ws = oracle.make_awq(K, N, gs, seed=5)
    awq = pkg.ops.make_packed(to_dev(wq, gpu), to_dev(wz, gpu), to_dev(ws, gpu), None, gs, 1)
    xs = {M: to_dev(oracle.make_x(M, K, seed=M), gpu) for M in (1, 2, 8, 18, 40, 300)}
    for M in xs:  # the largest workspace any call needs, reserved up front
        pkg.ops.reserve_workspace(gpu, int(pkg._lib.load().q4_workspace_bytes_perm(M, K, N)))

    def call(w, M, **kw):
        return lambda out: pkg.ops.linear(w, xs[M], None, out=out, **kw)

    calls = [
        call(plain, 1), call(plain, 2),      # accumulation cells
        call(plain, 8),                      # tickets
        call(plain, 18),                     # two MFMA row blocks
        call(plain, 40, path=2),             # split-K GEMM + reduction kernel
        call(plain, 300),
        call(seq, 1), call(seq, 8), call(seq, 300),   # fused gather, workspace gather, gather + GEMM
        call(act, 1), call(act, 8), call(awq, 1), call(awq, 8),
        lambda out: pkg.ops.linear_gate_up(plain, xs[1], "silu", out=out),
        lambda out: pkg.ops.linear_gate_up(seq, xs[2], "silu", out=out),
    ]
    capture_and_check(calls, gpu, between=lambda: [pkg.ops.linear(plain, xs[M]) for M in (1, 8, 40)])


def test_moe_block_under_graph_replay(pkg, oracle, gpu):
    E, k, H, I, gs = 4, 2, 1024, 512, 128
    rng = np.random.default_rng(0)

    def experts(K, N, act_order):
        parts = [oracle.make_gptq(K, N, gs, seed=10 + e + K, sym=False, act_order=act_order) for e in range(E)]
        stack = lambda i: to_dev(np.stack([p[i] for p in parts]), gpu)
        w = pkg.ops.make_packed_moe(stack(0), stack(1), stack(2), gs, stack(3) if act_order else None)
        return pkg.ops.make_sequential_moe(w) if act_order else w

    cases = []
    for act_order in (False, True):
        gu, dn = experts(H, 2 * I, act_order), experts(I, H, act_order)
        for T in (1, 5, 70):
            x = to_dev(oracle.make_x(T, H, seed=T), gpu)
            g = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(gpu)
            cases.append((gu, dn, x, g))

    def call(c):
        def fn(out):
            y = pkg.ops.moe_forward(c[0], c[1], c[2], c[3], k, True, "silu")
            if out is None:
                return y
            out.copy_(y)
            return out
        return fn

    capture_and_check([call(c) for c in cases], gpu,
                      between=lambda: pkg.ops.moe_forward(*cases[0][:4], k, True, "silu"))


@pytest.mark.parametrize("kind", ["act_order", "awq", "gptq"])
@pytest.mark.parametrize("M", [1, 16])
def test_first_forward_of_a_fresh_layer_is_capturable(pkg, oracle, gpu, kind, M):
    """Everything that is not the matmul (act-order test on g_idx, validation, launch plan,
    workspace) happens when the layer is built: its very first forward can be recorded into a
    HIP graph, and every replay (with eager work and synchronizations in between) returns the
    eager result bit for bit."""
    K, N, gs = 2048, 1024, 128
    if kind == "awq":
        qw, qz, sc = oracle.make_awq(K, N, gs, seed=3)
        build = lambda: pkg.WQLinear(4, gs, to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None)
    else:
        qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=4, sym=False, act_order=(kind == "act_order"))
        g = to_dev(gi, gpu) if gi is not None else (torch.arange(K, device=gpu) // gs).to(torch.int32)
        build = lambda: pkg.QuantLinear(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), g, None, 4, gs)
    x = to_dev(oracle.make_x(M, K, seed=M), gpu)
    want = build()(x).clone()  # eager result of an identical layer
    layer = build()            # fresh: has never run
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = layer(x)
    for i in range(3):
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), (kind, M, i)
        _ = layer(x + 1.0)  # eager work between the replays
        torch.cuda.synchronize()


def test_replay_after_the_workspace_grew_does_not_touch_freed_memory(pkg, oracle, gpu):
    """A graph captured with a small workspace keeps its address.  When a larger layer makes the
    shared workspace grow afterwards, the old buffer must stay allocated: replays write tickets,
    cells and partial sums there, and tensors allocated in between must not change."""
    ops = pkg.ops
    saved = dict(ops._workspaces)
    ops._workspaces.clear()  # this test starts from no workspace at all
    try:
        qw, qz, sc, _ = oracle.make_gptq(4096, 1024, 128, seed=31, sym=False)
        small = ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
        small.prepare(rows=(4,))
        x = to_dev(oracle.make_x(4, 4096, seed=2), gpu)
        eager = ops.linear(small, x)
        out = torch.empty_like(eager)
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                ops.linear(small, x, None, out=out)
        torch.cuda.synchronize()
        used = ops._workspaces[(gpu.index, ops.SHARED)]
        # a larger layer, planned for many rows: the shared workspace is replaced by a bigger one
        g = torch.Generator(device=gpu).manual_seed(5)
        big = ops.make_packed(
            torch.randint(-(2**31), 2**31 - 1, (14336 // 8, 4096), dtype=torch.int64, device=gpu, generator=g).to(torch.int32),
            torch.full((112, 512), 0x77777777, dtype=torch.int32, device=gpu),
            (torch.rand((112, 4096), device=gpu, generator=g) * 0.019 + 0.001).half(), None, 128, 0)
        big.prepare(max_rows=1024)
        assert ops._workspaces[(gpu.index, ops.SHARED)] is not used, "the workspace did not grow: the test shows nothing"
        assert any(t is used for t in ops._retired_workspaces)
        # memory the allocator would hand out if the old buffer had been freed
        del used
        torch.cuda.empty_cache()
        fillers = [torch.full((1 << 20,), 7, dtype=torch.int32, device=gpu) for _ in range(8)]
        torch.cuda.synchronize()
        for _ in range(3):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
        for f in fillers:
            assert bool((f == 7).all())
    finally:
        ops._workspaces.clear()
        ops._workspaces.update(saved)
