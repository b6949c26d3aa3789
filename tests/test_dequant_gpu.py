"""GPU parity: the HIP dequant kernel must reproduce the oracle's W bit for bit."""

import numpy as np
import pytest
import torch

from tests.util import bits_of, to_dev

pytestmark = pytest.mark.gpu

GPTQ_CASES = [
    # K, N, groupsize, sym, act_order
    (128, 64, 128, True, False),
    (256, 128, 32, False, False),
    (512, 256, 64, False, True),
    (4096, 4096, 128, True, False),   # BASELINE.json configs[0] shape
    (1024, 264, 128, False, False),   # N multiple of 8 only
    (1000, 64, 40, False, False),     # K multiple of 8 only, odd groupsize
    (2048, 512, -1, False, False),    # one group
    (8192, 1024, 128, False, True),   # act-order, 70B-like K
]


def _bits(w):
    return w.view(np.uint16) if w.dtype == np.float16 else w


@pytest.mark.parametrize("K,N,gs,sym,act", GPTQ_CASES)
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_dequant_gptq_bit_exact(pkg, oracle, gpu, K, N, gs, sym, act, dtype):
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=K + N, sym=sym, act_order=act)
    ref = oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    got = bits_of(pkg.ops.dequantize(pk, tdt))
    assert got.shape == (K, N)
    assert np.array_equal(got, _bits(ref))


@pytest.mark.parametrize("K,N,gs", [(128, 64, 128), (256, 72, 32), (4096, 14336, 128), (14336, 4096, 128), (512, 512, -1)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_dequant_awq_bit_exact(pkg, oracle, gpu, K, N, gs, dtype):
    qw, qz, sc = oracle.make_awq(K, N, gs, seed=K * 3 + N)
    ref = oracle.dequant_awq(qw, qz, sc, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 1)
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    got = bits_of(pkg.ops.dequantize(pk, tdt))
    assert np.array_equal(got, _bits(ref))


def test_dequant_extreme_scales(pkg, oracle, gpu):
    """Scales that push products into fp16 subnormals and up to the largest finite value."""
    K, N, gs = 256, 64, 128
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=5, sym=False)
    sc = sc.copy()
    sc[0, :16] = np.float16(6e-8)      # smallest subnormal region
    sc[0, 16:32] = np.float16(3e-6)
    sc[1, :16] = np.float16(4000.0)    # 15 * 4000 = 60000 < 65504
    sc[1, 16:32] = np.float16(0.0)
    ref = oracle.dequant_gptq(qw, qz, sc, None, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    got = bits_of(pkg.ops.dequantize(pk, torch.float16))
    assert np.array_equal(got, ref.view(np.uint16))
