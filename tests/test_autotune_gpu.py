"""Measured launch plans (ops.autotune) and the Warmup hook that runs them: a tuned plan computes
the same result as the library's own choice, stays capturable, and the hook sizes the shared
workspace for the row count it is given."""
import numpy as np
import pytest
import torch

from tests.util import max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _weights(pkg, oracle, gpu, K, N, n, seed=0):
    out = []
    for i in range(n):
        qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=seed + i, sym=False)
        out.append((pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0),
                    oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")))
    return out


def test_candidates_are_launchable_and_agree_with_the_default(pkg, oracle, gpu):
    (pk, w), = _weights(pkg, oracle, gpu, 4096, 2048, 1, seed=11)
    for M in (1, 3, 4, 16):
        cands = pkg.ops.decode_candidates(pk, M)
        assert cands, "the short-launch kernel takes this weight: there must be candidates"
        x = oracle.make_x(M, 4096, seed=M)
        y32, _ = oracle.linear_forward(x, w, None, "f16")
        for cfg in cands:
            got = to_f32(pkg.ops.linear(pk, to_dev(x, gpu), None, gemv_config=cfg))
            assert max_rel_err(got, y32) <= 2e-3, (M, cfg)


def test_no_candidates_where_no_decode_kernel_or_no_alternative(pkg, oracle, gpu):
    (pk, _), = _weights(pkg, oracle, gpu, 2048, 1024, 1, seed=3)
    assert pkg.ops.decode_candidates(pk, 2048) == []  # prefill
    qw, qz, sc = oracle.make_awq(1024, 512, 128, seed=1)
    awq = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 1)
    assert pkg.ops.decode_candidates(awq, 1) == []


def test_autotune_keeps_results_and_capturability(pkg, oracle, gpu):
    ws = _weights(pkg, oracle, gpu, 4096, 2048, 3, seed=21)
    packed = [pk for pk, _ in ws]
    for pk in packed:
        pk.prepare()
    report = pkg.ops.autotune(packed, rows=(1, 4, 8))
    assert set(report) == {(4096, 2048, 128, 1), (4096, 2048, 128, 4), (4096, 2048, 128, 8)}
    for (cfg, base_us, best_us) in report.values():
        assert cfg is None or (len(cfg) == 4 and best_us <= base_us)
    for M in (1, 4, 8):
        plans = {pk.plan(M, 0)[2] for pk in packed}
        assert len(plans) == 1, "every weight of the group gets the same plan"
        x = oracle.make_x(M, 4096, seed=M + 5)
        xt = to_dev(x, gpu)
        for pk, w in ws:
            y32, _ = oracle.linear_forward(x, w, None, "f16")
            eager = pkg.ops.linear(pk, xt)
            assert max_rel_err(to_f32(eager), y32) <= 2e-3
            # the tuned call inside a graph: nothing allocates, replays agree with eager bit for bit
            out = torch.empty_like(eager)
            side = torch.cuda.Stream()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    pkg.ops.linear(pk, xt, None, out=out)
            torch.cuda.synchronize()
            for _ in range(3):
                out.zero_()
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(out, eager)


def test_warmup_hook_sizes_the_workspace_and_tunes(pkg, oracle, gpu, monkeypatch):
    qw, qz, sc, _ = oracle.make_gptq(2048, 4096, 128, seed=4, sym=False)
    weight = pkg.GPTQWeight(qweight=to_dev(qw, gpu), qzeros=to_dev(qz, gpu), scales=to_dev(sc, gpu), g_idx=None,
                            bits=4, groupsize=128, use_awq_kernel=False, use_exllama=True)
    layer = pkg.get_linear(weight, None)
    pkg.set_device(gpu)
    assert pkg.create_exllama_buffers(3000) is None
    shared = pkg.ops._workspaces[(gpu.index, pkg.ops.SHARED)]
    for M in (1, 16, 3000):
        assert shared.numel() >= layer._packed.plan(M, 0)[1]
    assert any(k[:3] == (2048, 4096, 128) for k in pkg.ops.last_autotune_report)
    w = oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")
    x = oracle.make_x(2, 2048, seed=9)
    y32, _ = oracle.linear_forward(x, w, None, "f16")
    assert max_rel_err(to_f32(layer(to_dev(x, gpu))), y32) <= 2e-3
    monkeypatch.setenv("Q4_AUTOTUNE", "0")
    pkg.ops.last_autotune_report = {}
    pkg.create_exllama_buffers(64)
    assert pkg.ops.last_autotune_report == {}
