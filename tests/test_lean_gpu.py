"""The instruction-lean contiguous-group decode kernel (gemv_gptq_lean_kernel) against the oracle,
forced through explicit decompositions (`words = 0` in the tuned entry point selects it):
every row-count variant (1, 2, 4, 8, 16 rows padded), both dtypes, workgroup-slab and per-wave
activation staging, split-K through cells and tickets, accumulation periods that end inside and
outside the load ring, and one-hot rows that must read the dequantized weights back bit for bit."""
import numpy as np
import pytest
import torch

from tests.util import bits_of, max_rel_err, to_dev, to_f32
from tests.test_linear_gpu import _run

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 11, 16, 17, 33])
@pytest.mark.parametrize("cfg", [(1, 1, 1, 0), (1, 4, 2, 0), (2, 4, 1, 0), (1, 8, 2, 0), (1, 16, 1, 0), (2, 8, 1, 0), (1, 2, 8, 0), (4, 4, 1, 0)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_lean_small(pkg, oracle, gpu, M, cfg, dtype):
    try:
        _run(pkg, oracle, gpu, 2048, 1024, 128, M, dtype=dtype, sym=False, bias=(M % 2 == 0), cfg=cfg, seed=M + sum(cfg))
    except pkg._lib.Q4Error as e:
        if "LDS" not in str(e):
            raise
        pytest.skip("every wave stages its own activations: this decomposition does not fit LDS")


@pytest.mark.parametrize("K,N,cfg", [(4096, 4096, (1, 8, 4, 0)), (4096, 6144, (1, 8, 2, 0)), (4096, 28672, (1, 8, 1, 0)),
                                     (14336, 4096, (1, 8, 7, 0)), (14336, 4096, (1, 16, 7, 0)), (4096, 28672, (1, 16, 1, 0)),
                                     (11008, 4096, (1, 8, 3, 0)), (8192, 1024, (1, 16, 4, 0))])
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16])
def test_lean_llama(pkg, oracle, gpu, K, N, cfg, M):
    _run(pkg, oracle, gpu, K, N, 128, M, cfg=cfg, seed=K // 64 + N // 64 + M)


@pytest.mark.parametrize("gs", [128, 256, 512, -1])
@pytest.mark.parametrize("M", [1, 3, 16])
def test_lean_groupsizes(pkg, oracle, gpu, gs, M):
    _run(pkg, oracle, gpu, 1024, 256, gs, M, sym=False, cfg=(1, 2, 2, 0), seed=gs + 100)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows", [1, 2, 4, 8, 16])
def test_lean_one_hot_reads_weights_back(pkg, oracle, gpu, dtype, rows):
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
    for cfg in [(1, 1, 1, 0), (1, 4, 2, 0), (2, 2, 1, 0)]:
        y = pkg.ops.linear(pk, x, None, gemv_config=cfg)
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(y), w[ks].view(np.uint16)), cfg


@pytest.mark.parametrize("chunks", [1, 2, 3, 5, 6, 9, 17, 18, 19, 33, 35])
@pytest.mark.parametrize("M", [1, 2, 4])
def test_lean_period_boundaries(pkg, oracle, gpu, chunks, M):
    """One wave walks the whole K: periods of 16 / 8 / 4 chunks that end inside the ring."""
    _run(pkg, oracle, gpu, chunks * 128, 128, 128, M, sym=False, cfg=(1, 1, 1, 0), seed=chunks + M)
    if chunks >= 4:
        _run(pkg, oracle, gpu, chunks * 128, 128, 128, M, sym=False, cfg=(1, 2, 2, 0), seed=chunks + M + 1)


@pytest.mark.parametrize("K,N", [(8192, 10240), (5120, 13824), (13824, 5120), (28672, 8192), (8192, 28672), (6656, 17920),
                                 (3584, 37888), (3072, 9216), (2048, 9216), (8192, 1280)])
def test_large_layer_decode_decompositions_picked(pkg, gpu, K, N):
    """The decompositions the picker takes for 4..16 rows on large layers (several column tiles
    around one slab, 1024-thread workgroups, splits of an uneven K deal): one-hot rows read the
    dequantized weights back bit for bit, and random activations agree with the prefill kernel."""
    g = torch.Generator(device=gpu).manual_seed(K + N)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K // 8, N), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    qzeros = torch.randint(-(2**31), 2**31 - 1, (K // 128, N // 8), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    scales = (torch.rand((K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    w = pkg.ops.make_packed(qweight, qzeros, scales, None, 128, 0)
    dense = pkg.ops.dequantize(w)
    rows = torch.randint(0, K, (16,), device=gpu, generator=g)
    for M in (1, 3, 4, 6, 9, 12, 16):
        assert pkg.ops.select_path(w, M) == "gemv"
        x = torch.zeros((M, K), dtype=torch.float16, device=gpu)
        x[torch.arange(M, device=gpu), rows[:M]] = 1.0
        assert torch.equal(pkg.ops.linear(w, x), dense[rows[:M]]), f"one-hot rows, M={M}"
        x = torch.randn((M, K), dtype=torch.float16, device=gpu, generator=g)
        y, ref = pkg.ops.linear(w, x).float(), pkg.ops.linear(w, x, path=2).float()
        err = float((y - ref).abs().max() / ref.abs().max())
        assert err <= 2e-3, f"M={M}: {err:.2e}"
