"""The short-launch decode kernel (gemv_gptq_direct_kernel: up to 16 rows, activations fetched
straight from global memory, the grid as the work decomposition) against the oracle, forced
through explicit decompositions (`words = -1` in the tuned entry point selects it; the tuple is
(unused, K waves per workgroup, workgroups along K, -1)): every row count, both dtypes, unsplit
and split K (fixed-point cells for fp16 rows, tickets for bf16), even and ragged K deals,
group sizes, and one-hot rows that must read the dequantized weights back bit for bit."""
import numpy as np
import pytest
import torch

from tests.util import bits_of, max_rel_err, to_dev, to_f32
from tests.test_linear_gpu import _run

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 11, 16])
@pytest.mark.parametrize("cfg", [(1, 1, 1, -1), (1, 4, 1, -1), (1, 8, 1, -1), (1, 2, 8, -1), (1, 4, 4, -1), (1, 1, 16, -1), (1, 8, 2, -1), (1, 3, 5, -1)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_direct_small(pkg, oracle, gpu, M, cfg, dtype):
    _run(pkg, oracle, gpu, 2048, 1024, 128, M, dtype=dtype, sym=False, bias=(M % 2 == 0), cfg=cfg, seed=M + sum(cfg))


@pytest.mark.parametrize("K,N,cfg", [(4096, 4096, (1, 4, 8, -1)), (4096, 4096, (1, 1, 8, -1)), (4096, 6144, (1, 4, 8, -1)),
                                     (4096, 28672, (1, 4, 1, -1)), (4096, 28672, (1, 8, 2, -1)), (14336, 4096, (1, 8, 7, -1)),
                                     (14336, 4096, (1, 4, 14, -1)), (14336, 4096, (1, 2, 14, -1)), (8192, 1024, (1, 8, 8, -1))])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 8, 16])
def test_direct_llama(pkg, oracle, gpu, K, N, cfg, M):
    _run(pkg, oracle, gpu, K, N, 128, M, cfg=cfg, seed=K // 64 + N // 64 + M)


@pytest.mark.parametrize("gs", [128, 256, 512, -1])
@pytest.mark.parametrize("M", [1, 3])
def test_direct_groupsizes(pkg, oracle, gpu, gs, M):
    _run(pkg, oracle, gpu, 1024, 256, gs, M, sym=False, cfg=(1, 2, 2, -1), seed=gs + 100)
    _run(pkg, oracle, gpu, 1024, 256, gs, M, sym=False, cfg=(1, 1, 1, -1), seed=gs + 101)


def test_direct_refuses_what_it_does_not_take(pkg, oracle, gpu):
    with pytest.raises(pkg._lib.Q4Error):  # groups of 384 rows: not 128 << s
        _run(pkg, oracle, gpu, 768, 256, 384, 1, cfg=(1, 1, 1, -1))
    with pytest.raises(pkg._lib.Q4Error):  # more wave slots than chunks
        _run(pkg, oracle, gpu, 1024, 256, 128, 1, cfg=(1, 3, 3, -1))
    with pytest.raises(pkg._lib.Q4Error):  # seventeen rows
        _run(pkg, oracle, gpu, 1024, 256, 128, 17, cfg=(1, 2, 1, -1))
    with pytest.raises(pkg._lib.Q4Error):  # act-order
        _run(pkg, oracle, gpu, 1024, 256, 128, 1, act=True, cfg=(1, 2, 1, -1))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows", [1, 2, 3, 4, 7, 16])
def test_direct_one_hot_reads_weights_back(pkg, oracle, gpu, dtype, rows):
    """x = rows of the identity: y must be the dequantized weight rows bit for bit."""
    K, N, gs = 1024, 512, 128
    bf = dtype == "bf16"
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=3, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    rng = np.random.default_rng(rows)
    ks = rng.choice(K, size=rows, replace=False)
    x = torch.zeros((rows, K), dtype=torch.bfloat16 if bf else torch.float16, device=gpu)
    for i, k in enumerate(ks):
        x[i, k] = 1.0
    cfgs = [(1, 1, 1, -1), (1, 4, 1, -1), (1, 4, 2, -1), (1, 1, 8, -1), (1, 3, 1, -1)]
    for cfg in cfgs:
        y = pkg.ops.linear(pk, x, None, gemv_config=cfg)
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(y), w[ks].view(np.uint16)), cfg


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [3, 4, 7, 16])
@pytest.mark.parametrize("cfg", [(1, 4, 8, -1), (1, 8, 4, -1), (1, 1, 14, -1), None])
def test_direct_split_k_is_reproducible_and_leaves_the_counters_zero(pkg, oracle, gpu, M, cfg, dtype):
    """Cells (fp16: wave 0 row by row up to three rows, the rows dealt to the waves beyond) and
    tickets (bf16): the same bits on every call, the oracle's result, counters back at zero.
    cfg None: the decomposition the plain call takes."""
    bf = dtype == "bf16"
    qw, qz, sc, _ = oracle.make_gptq(4096, 4096, 128, seed=8, sym=False)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    x = oracle.make_x(M, 4096, seed=5, dtype=dtype)
    xd = to_dev(x, gpu, bf16=bf)
    a = pkg.ops.linear(pk, xd, None, gemv_config=cfg, path=1)
    b = pkg.ops.linear(pk, xd, None, gemv_config=cfg, path=1)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    for ws in pkg.ops._workspaces.values():
        assert int(ws[: pkg._lib.WORKSPACE_COUNTER_BYTES].sum().item()) == 0
    ref = oracle.matmul_fp32(oracle.to_f32(x, dtype), oracle.to_f32(oracle.dequant_gptq(qw, qz, sc, None, 128, dtype), dtype))
    assert max_rel_err(to_f32(a), ref) <= (8e-3 if bf else 2e-3)


@pytest.mark.parametrize("M,cfg", [(1, (1, 4, 8, -1)), (2, (1, 2, 1, -1)), (3, (1, 4, 4, -1)), (4, (1, 4, 2, -1)), (16, (1, 8, 1, -1)), (9, (1, 4, 4, -1))])
@pytest.mark.parametrize("poison", ["+inf", "-inf", "nan", "+inf,-inf"])
def test_direct_non_finite_activations_keep_their_class(pkg, oracle, gpu, M, cfg, poison):
    """An inf or NaN activation: every output is NaN, +inf or -inf exactly where fp32 arithmetic on
    the dequantized weights gives that class (the wave that meets the poisoned chunk redoes its K
    range with the zero point taken out before the MFMA), and the other rows stay correct."""
    K, N = 4096, 1024
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=77, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    x = oracle.make_x(M, K, seed=M).copy()
    vals = {"+inf": np.inf, "-inf": -np.inf, "nan": np.nan}
    for i, name in enumerate(poison.split(",")):
        x[M - 1, 100 + 1500 * i] = np.float16(vals[name])
    with np.errstate(invalid="ignore", over="ignore"):
        ref = x.astype(np.float32) @ w.astype(np.float32)
    got = pkg.ops.linear(pk, to_dev(x, gpu), None, gemv_config=cfg).float().cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isposinf(got), np.isposinf(ref))
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    if M > 1:
        clean = np.abs(got[: M - 1] - ref[: M - 1]).max() / np.abs(ref[: M - 1]).max()
        assert clean <= 2e-3
