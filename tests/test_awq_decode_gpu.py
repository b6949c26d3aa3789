"""The AWQ-layout decode kernel that feeds the stored words to the matrix core
(gemv_awq_diag_kernel), forced through explicit decompositions (`words = 0` in the tuned entry
point selects it for up to 8 rows): every row count 1..8, both dtypes, group sizes 32..256 and
one group per column, split-K through cells and tickets, several column waves, and one-hot rows
that must read the dequantized weights back bit for bit.  The kernel it replaces for these row
counts (`words = 4`) must agree with it."""
import numpy as np
import pytest
import torch

from tests.util import bits_of, to_dev, to_f32
from tests.test_linear_gpu import _run

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("cfg", [(1, 1, 1, 0), (1, 4, 2, 0), (2, 4, 1, 0), (1, 8, 2, 0), (2, 2, 4, 0), (1, 2, 8, 0)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_awq_words_as_stored_small(pkg, oracle, gpu, M, cfg, dtype):
    _run(pkg, oracle, gpu, 2048, 1024, 128, M, dtype=dtype, layout="awq", bias=(M % 2 == 0), cfg=cfg, seed=M + sum(cfg))


@pytest.mark.parametrize("K,N,cfg", [(4096, 4096, (1, 4, 8, 0)), (4096, 14336, (1, 8, 4, 0)), (14336, 4096, (1, 8, 14, 0)),
                                     (4096, 6144, (1, 4, 8, 0)), (11008, 4096, (1, 4, 7, 0)), (4096, 28672, (2, 4, 4, 0))])
@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_awq_words_as_stored_model_shapes(pkg, oracle, gpu, K, N, cfg, M):
    _run(pkg, oracle, gpu, K, N, 128, M, layout="awq", cfg=cfg, seed=K // 64 + N // 64 + M)


@pytest.mark.parametrize("gs", [32, 64, 128, 256, -1])
@pytest.mark.parametrize("M", [1, 3, 8])
def test_awq_words_as_stored_groupsizes(pkg, oracle, gpu, gs, M):
    _run(pkg, oracle, gpu, 1024, 512, gs, M, layout="awq", cfg=(1, 2, 2, 0), seed=gs + 100)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows", [1, 2, 4, 5, 8])
def test_awq_one_hot_reads_weights_back(pkg, oracle, gpu, dtype, rows):
    """x = rows of the identity: y must be the dequantized weight rows bit for bit."""
    K, N, gs = 1024, 512, 128
    bf = dtype == "bf16"
    qw, qz, sc = oracle.make_awq(K, N, gs, seed=5)
    w = oracle.dequant_awq(qw, qz, sc, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 1)
    rng = np.random.default_rng(rows)
    ks = rng.choice(K, size=rows, replace=False)
    x = torch.zeros((rows, K), dtype=torch.bfloat16 if bf else torch.float16, device=gpu)
    for i, k in enumerate(ks):
        x[i, k] = 1.0
    for cfg in [(1, 1, 1, 0), (1, 4, 2, 0), (2, 2, 1, 0)]:
        y = pkg.ops.linear(pk, x, None, gemv_config=cfg)
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(y), w[ks].view(np.uint16)), cfg


@pytest.mark.parametrize("M", [1, 4, 8])
def test_awq_kernels_agree_and_default_takes_the_new_one(pkg, oracle, gpu, M):
    """Both AWQ decode kernels on the same decomposition, and the library's own choice."""
    K, N = 4096, 2048
    qw, qz, sc = oracle.make_awq(K, N, 128, seed=M)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 1)
    x = to_dev(oracle.make_x(M, K, seed=M + 3), gpu)
    new = to_f32(pkg.ops.linear(pk, x, None, gemv_config=(1, 4, 4, 0)))
    old = to_f32(pkg.ops.linear(pk, x, None, gemv_config=(1, 4, 4, 4)))
    auto = to_f32(pkg.ops.linear(pk, x, None))
    scale = np.abs(old).max()
    assert np.abs(new - old).max() <= 2e-3 * scale
    assert np.abs(auto - old).max() <= 2e-3 * scale
