"""The AWQ-layout prefill kernel that unpacks the checkpoint words in registers
(gemm_awq_direct_kernel: N a multiple of 256, groups of 64 rows or more): every row tile (32, 64,
96 rows), partial last tiles, both dtypes, bias, split-K grids (few column tiles, long K), the
eight-wave variant (one workgroup per CU) and the four-wave variant with several workgroups per
CU, group sizes 64 .. one group, and one-hot rows that must read the dequantized weights back
bit for bit at every tile position.  AWQ weights the kernel does not take (groups of 32 rows,
N = 128 mod 256) must still run on the kernel that unpacks through LDS."""
import numpy as np
import pytest
import torch

from tests.util import bits_of, to_dev
from tests.test_linear_gpu import _run

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M", [9, 20, 32, 33, 50, 64, 65, 96, 100, 128, 130, 192, 200, 300])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_awq_prefill_row_tiles(pkg, oracle, gpu, M, dtype):
    """Row counts on both sides of every tile boundary; K long enough for split-K at small M."""
    _run(pkg, oracle, gpu, 2048, 512, 128, M, dtype=dtype, layout="awq", bias=(M % 2 == 0), path=2, seed=M)


@pytest.mark.parametrize("K,N,M", [(4096, 4096, 16), (4096, 4096, 700), (14336, 4096, 40), (4096, 14336, 100),
                                   (4096, 14336, 1000), (1024, 8192, 1500), (11008, 4096, 96), (4096, 11008 + 256, 64)])
def test_awq_prefill_grids(pkg, oracle, gpu, K, N, M):
    """Split-K (few tiles), eight waves in two K groups (at most one workgroup per CU), four waves
    with several workgroups per CU, K tile counts that are odd or do not divide by the split."""
    _run(pkg, oracle, gpu, K, N, 128, M, layout="awq", path=2, bias=(M == 100), seed=K // 128 + M)


@pytest.mark.parametrize("gs", [64, 128, 256, 1024, -1])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_awq_prefill_groupsizes(pkg, oracle, gpu, gs, dtype):
    _run(pkg, oracle, gpu, 1024, 512, gs, 150, dtype=dtype, layout="awq", path=2, seed=gs + 3)


@pytest.mark.parametrize("gs,N", [(32, 512), (128, 384)])
def test_awq_prefill_falls_back_to_the_lds_kernel(pkg, oracle, gpu, gs, N):
    _run(pkg, oracle, gpu, 1024, N, gs, 150, layout="awq", path=2, seed=gs + N)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [24, 64, 96, 333, 1024])
def test_awq_prefill_one_hot_reads_weights_back(pkg, oracle, gpu, dtype, M):
    """x = rows of the identity (random K positions): y must be the dequantized rows bit for bit."""
    K, N, gs = 2048, 1024, 128
    bf = dtype == "bf16"
    qw, qz, sc = oracle.make_awq(K, N, gs, seed=M)
    w = oracle.dequant_awq(qw, qz, sc, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 1)
    ks = np.random.default_rng(M).integers(0, K, size=M)
    x = torch.zeros((M, K), dtype=torch.bfloat16 if bf else torch.float16, device=gpu)
    x[torch.arange(M, device=gpu), torch.from_numpy(ks).to(gpu)] = 1.0
    y = pkg.ops.linear(pk, x, None, path=2)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(y), w[ks].view(np.uint16))


@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_awq_prefill_mistral_one_hot_full_size(pkg, gpu, K, N, dtype):
    """Full Mistral-7B shapes at prefill sizes: one-hot rows against the library's own dequantize
    (bit-exact against the oracle in the dequant tests), M = 512 and 2048."""
    g = torch.Generator(device=gpu).manual_seed(K + N)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K, N // 8), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    qzeros = torch.randint(-(2**31), 2**31 - 1, (K // 128, N // 8), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    scales = (torch.rand((K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    w = pkg.ops.make_packed(qweight, qzeros, scales, None, 128, 1)
    dense = pkg.ops.dequantize(w, dtype)
    for M in (512, 2048):
        rows = torch.randint(0, K, (M,), device=gpu, generator=g)
        x = torch.zeros((M, K), dtype=dtype, device=gpu)
        x[torch.arange(M, device=gpu), rows] = 1.0
        y = pkg.ops.linear(w, x)
        assert torch.equal(y, dense[rows]), f"M={M}"
        del x, y


def test_awq_prefill_split_k_is_deterministic(pkg, oracle, gpu):
    K, N, M = 8192, 512, 48
    qw, qz, sc = oracle.make_awq(K, N, 128, seed=4)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 1)
    x = torch.randn((M, K), device=gpu, dtype=torch.float16)
    ys = [pkg.ops.linear(pk, x, None, path=2).clone() for _ in range(4)]
    for y in ys[1:]:
        assert torch.equal(y, ys[0])
