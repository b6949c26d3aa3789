"""GPU parity at the full sizes of the benchmark configurations that the small-shape tests do
not reach: bf16 prefill at M = 512 / 2048 / 4096 on the four Llama-3-8B projections, act-order
at the Llama-3-70B shapes up to M = 1024 (checkpoint-order kernels and the layers' own route),
and the AWQ row sweep on the Mistral-7B shapes.

The HIP path runs the whole problem; the oracle (NumPy, fp32 accumulation over the bit-exact
dequantized weights) is evaluated on a random subset of the activation rows, which keeps the
host side to seconds.  Tolerances: max|y - ref| / max|ref| <= 2e-3 in fp16; bf16 outputs are
compared at 8e-3 (the bf16 output rounding alone is 2^-8 per element).
"""

import numpy as np
import pytest
import torch

from tests.util import max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu

TOL = 2e-3
TOL_BF16 = 8e-3
LLAMA3_8B = [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)]


def _rows_check(oracle, x_np, w, got, dtype, rows):
    """Compare the rows `rows` of the device result with the oracle's on the same inputs."""
    y32, _ = oracle.linear_forward(np.ascontiguousarray(x_np[rows]), w, None, dtype)
    g = to_f32(got[torch.as_tensor(rows, device=got.device)])
    assert np.isfinite(g).all()
    err = max_rel_err(g, y32)
    assert err <= (TOL_BF16 if dtype == "bf16" else TOL), f"max rel err {err:.3e}"


def _x(oracle, M, K, seed, dtype, gpu):
    x = oracle.make_x(M, K, seed=seed, dtype=dtype)
    return x, to_dev(x, gpu, bf16=(dtype == "bf16"))


@pytest.mark.parametrize("K,N", LLAMA3_8B)
def test_cfg3_bf16_prefill_full_sizes(pkg, oracle, gpu, K, N):
    """BASELINE.json configs[2]: bf16 activations, M in {512, 2048, 4096}, every projection."""
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=K // 128 + N // 128)
    w = oracle.dequant_gptq(qw, qz, sc, None, 128, "bf16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    rng = np.random.default_rng(K + N)
    for M in (512, 2048, 4096):
        x, xt = _x(oracle, M, K, M, "bf16", gpu)
        assert pkg.ops.select_path(pk, M, torch.bfloat16) == "gemm"
        got = pkg.ops.linear(pk, xt, None)
        torch.cuda.synchronize()
        assert got.shape == (M, N) and got.dtype == torch.bfloat16
        _rows_check(oracle, x, w, got, "bf16", np.sort(rng.choice(M, size=48, replace=False)))


@pytest.mark.parametrize("K,N", LLAMA3_8B)
def test_cfg3_fp16_prefill_m4096(pkg, oracle, gpu, K, N):
    """The same shapes in fp16 at the largest prefill size (max_batch_prefill_tokens = 4096)."""
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=K // 64 + N // 64, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    x, xt = _x(oracle, 4096, K, 4096, "f16", gpu)
    got = pkg.ops.linear(pk, xt, None)
    torch.cuda.synchronize()
    _rows_check(oracle, x, w, got, "f16", np.sort(np.random.default_rng(N).choice(4096, size=48, replace=False)))


@pytest.mark.parametrize("K,N", LLAMA3_8B)
def test_full_size_properties_bf16_and_prefill_sizes(pkg, gpu, K, N):
    """Size-independent properties in bf16 and at prefill sizes: one-hot rows read the bf16
    dequantized weights back bit for bit through the prefill kernel at M = 512 / 2048 / 4096
    (every tile variant), decode and prefill kernels agree on random bf16 activations."""
    g = torch.Generator(device=gpu).manual_seed(K * 3 + N)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K // 8, N), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    qzeros = torch.randint(-(2**31), 2**31 - 1, (K // 128, N // 8), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    scales = (torch.rand((K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    w = pkg.ops.make_packed(qweight, qzeros, scales, None, 128, 0)
    for dtype in (torch.bfloat16, torch.float16):
        dense = pkg.ops.dequantize(w, dtype)  # bit-exact against the oracle in the dequant tests
        for M in (512, 2048, 4096):
            rows = torch.randint(0, K, (M,), device=gpu, generator=g)
            x = torch.zeros((M, K), dtype=dtype, device=gpu)
            x[torch.arange(M, device=gpu), rows] = 1.0
            y = pkg.ops.linear(w, x)
            assert torch.equal(y, dense[rows]), f"one-hot rows, M={M}, {dtype}"
            del x, y
    a = torch.randn((16, K), device=gpu, dtype=torch.bfloat16, generator=g)
    ya = pkg.ops.linear(w, a, path=1).float()
    ga = pkg.ops.linear(w, a, path=2).float()
    assert float((ya - ga).abs().max()) <= TOL_BF16 * float(ya.abs().max())


@pytest.mark.parametrize("K,N", [(8192, 10240), (28672, 8192)])
def test_cfg4_act_order_llama70b_all_m(pkg, oracle, gpu, K, N):
    """BASELINE.json configs[3]: desc_act with a random row permutation at the Llama-3-70B
    shapes, M in {1, 16, 1024}: the kernels that read the checkpoint layout through g_idx, and
    the route the layers take (rows in group order, activations read through the permutation)."""
    qw, qz, sc, gi = oracle.make_gptq(K, N, 128, seed=K // 512 + 3, act_order=True)
    w = oracle.dequant_gptq(qw, qz, sc, gi, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), 128, 0)
    seq = pkg.ops.make_sequential(pk)
    assert seq is not None and seq.perm is not None
    rng = np.random.default_rng(K)
    for M in (1, 16, 1024):
        x, xt = _x(oracle, M, K, M + 5, "f16", gpu)
        rows = np.sort(rng.choice(M, size=min(M, 32), replace=False))
        for weight in (pk, seq):
            got = pkg.ops.linear(weight, xt, None)
            torch.cuda.synchronize()
            _rows_check(oracle, x, w, got, "f16", rows)


@pytest.mark.parametrize("K,N", [(8192, 10240), (28672, 8192)])
def test_cfg4_layers_default_route_llama70b(pkg, oracle, gpu, K, N):
    """The module a loader would build for an act-order checkpoint (GPTQWeight.get_linear), at the
    70B shapes: its forward against the oracle, whatever route the layer takes inside."""
    qw, qz, sc, gi = oracle.make_gptq(K, N, 128, seed=K // 256 + 1, act_order=True)
    w = oracle.dequant_gptq(qw, qz, sc, gi, 128, "f16")
    weight = pkg.GPTQWeight(qweight=to_dev(qw, gpu), qzeros=to_dev(qz, gpu), scales=to_dev(sc, gpu), g_idx=to_dev(gi, gpu),
                            bits=4, groupsize=128, use_awq_kernel=False, use_exllama=True)
    layer = pkg.get_linear(weight, None)
    rng = np.random.default_rng(N)
    for M in (1, 16, 1024):
        x, xt = _x(oracle, M, K, M + 9, "f16", gpu)
        got = layer(xt)
        torch.cuda.synchronize()
        _rows_check(oracle, x, w, got, "f16", np.sort(rng.choice(M, size=min(M, 32), replace=False)))


@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
@pytest.mark.parametrize("M", [8, 32, 64, 128, 256])
def test_cfg5_awq_m_sweep_mistral(pkg, oracle, gpu, K, N, M):
    """BASELINE.json configs[4]: AWQ layout, asymmetric zeros, Mistral-7B shapes, the row counts
    between the decode sizes and 256 (1, 2, 4, 16 run in test_linear_gpu.py)."""
    qw, qz, sc = oracle.make_awq(K, N, 128, seed=K // 256 + M)
    w = oracle.dequant_awq(qw, qz, sc, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 1)
    x, xt = _x(oracle, M, K, M, "f16", gpu)
    got = pkg.ops.linear(pk, xt, None)
    torch.cuda.synchronize()
    _rows_check(oracle, x, w, got, "f16", np.arange(M) if M <= 64 else np.sort(np.random.default_rng(M).choice(M, size=64, replace=False)))


@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_cfg5_wqlinear_module_mistral(pkg, oracle, gpu, K, N):
    """WQLinear as the loader builds it, whatever layout it runs on inside, M = 1 .. 256."""
    qw, qz, sc = oracle.make_awq(K, N, 128, seed=N // 256)
    w = oracle.dequant_awq(qw, qz, sc, 128, "f16")
    layer = pkg.WQLinear(4, 128, to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None)
    assert tuple(layer.qweight.shape) == (K, N // 8)  # the checkpoint tensor keeps its layout
    for M in (1, 2, 4, 8, 16, 32, 64, 128, 256):
        x, xt = _x(oracle, M, K, M + 1, "f16", gpu)
        got = layer(xt)
        torch.cuda.synchronize()
        _rows_check(oracle, x, w, got, "f16", np.arange(min(M, 24)))
    assert tuple(layer.qweight.shape) == (K, N // 8)


def test_prefill_activation_matrix_beyond_4gb_runs_in_row_blocks(pkg, gpu):
    """The prefill kernel addresses activations through 32-bit byte offsets; a matrix of more than
    4 GB goes through the launcher's row blocks.  Rows on both sides of the block boundary and at
    both ends must agree with what the same rows give on their own (a split-K launch there: same
    fp16 weights, another fp32 summation order)."""
    K, N = 4096, 128
    M = 524032 + 100  # the first block is 524032 rows at K = 4096
    g = torch.Generator(device=gpu).manual_seed(11)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K // 8, N), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    qzeros = torch.randint(-(2**31), 2**31 - 1, (K // 128, N // 8), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    scales = (torch.rand((K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    w = pkg.ops.make_packed(qweight, qzeros, scales, None, 128, 0)
    x = torch.empty((M, K), dtype=torch.float16, device=gpu)
    x.normal_(generator=g)
    y = pkg.ops.linear(w, x)
    torch.cuda.synchronize()
    for lo, hi in [(0, 200), (524032 - 150, 524032 + 100), (M - 100, M)]:
        ref = pkg.ops.linear(w, x[lo:hi].contiguous(), path=2).float()
        err = float((y[lo:hi].float() - ref).abs().max() / ref.abs().max())
        assert err <= TOL, (lo, hi, err)
    del x, y
    torch.cuda.empty_cache()
