"""Gated-MLP epilogue, act(x @ gate) * (x @ up), against the oracle.

The oracle applies eager PyTorch's roundings (linear output rounded to the activation dtype,
activation evaluated in fp32 and rounded, product rounded); the kernels do the same in their
epilogue.  Bar: max|y - ref| / max|ref| <= 2e-3 (fp16), 8e-3 (bf16 output
rounding alone is 3.9e-3).
"""

import numpy as np
import pytest
import torch

from tests.util import max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu

TOL = 2e-3
TOL_BF16 = 8e-3


def _case(pkg, oracle, gpu, K, N, gs, M, act="silu", dtype="f16", layout="gptq", act_order=False, bias=False,
          fused=None, seed=0):
    bf = dtype == "bf16"
    if layout == "gptq":
        qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=seed, sym=False, act_order=act_order)
        w = oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype)
        lay = 0
    else:
        qw, qz, sc = oracle.make_awq(K, N, gs, seed=seed)
        gi = None
        w = oracle.dequant_awq(qw, qz, sc, gs, dtype)
        lay = 1
    # scale x so that the gate values spread over the activation's curved region
    x = oracle.make_x(M, K, seed=seed, dtype=dtype)
    b = None
    if bias:
        bf32 = np.random.default_rng(seed + 1).standard_normal(N).astype(np.float32)
        b = bf32.astype(np.float16) if not bf else oracle.f32_to_bf16_bits(bf32)
    exact, want = oracle.gate_up_forward(x, w, act, b, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, lay)
    got = pkg.ops.linear_gate_up(pk, to_dev(x, gpu, bf16=bf), act, to_dev(b, gpu, bf16=bf), fused=fused)
    torch.cuda.synchronize()
    assert got.shape == (M, N // 2) and got.dtype == (torch.bfloat16 if bf else torch.float16)
    g = to_f32(got)
    assert np.isfinite(g).all()
    ref = oracle.to_f32(want, dtype)
    err = max_rel_err(g, ref)
    assert err <= (TOL_BF16 if bf else TOL), f"max rel err {err:.3e}"
    # and against the unrounded fp32 chain
    assert max_rel_err(g, exact) <= (TOL_BF16 if bf else TOL)
    return g


@pytest.mark.parametrize("M", [1, 2, 3, 8, 16])
def test_decode_llama3_8b_gate_up(pkg, oracle, gpu, M):
    # the fused kernel is offered for one and two rows; more rows take the two-kernel route
    _case(pkg, oracle, gpu, 4096, 28672, 128, M, fused=True if M <= 2 else None, seed=M)


@pytest.mark.parametrize("K,N,gs", [(1024, 256, 128), (2048, 1024, 128), (1024, 512, 32), (1024, 512, 64),
                                    (2048, 512, 256), (1024, 384, -1)])
@pytest.mark.parametrize("M", [1, 2, 5])
def test_decode_small_shapes_split_k(pkg, oracle, gpu, K, N, gs, M):
    """Few column tiles: the K range is split over workgroups and the activation is applied by
    the workgroup that combines the partials."""
    # groups smaller than a 128-row chunk have no fused kernel: those take the two-kernel route
    _case(pkg, oracle, gpu, K, N, gs, M, bias=True, fused=True if (gs == -1 or gs >= 128) and M <= 2 else None,
          seed=K // 64 + N + M)


@pytest.mark.parametrize("M", [1, 2])
def test_decode_fused_ragged_k_partition(pkg, oracle, gpu, M):
    """43 chunks of 128 rows do not divide over the wave slots of the fused kernel."""
    _case(pkg, oracle, gpu, 43 * 128, 512, 128, M, fused=True, seed=M + 5)


@pytest.mark.parametrize("act", ["silu", "gelu_tanh", "gelu", "gelu_fast", "gelu_pytorch_tanh"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_activations_decode_and_prefill(pkg, oracle, gpu, act, dtype):
    oracle_act = {"gelu_fast": "gelu_tanh", "gelu_pytorch_tanh": "gelu_tanh"}.get(act, act)
    for M in (2, 192):
        bf = dtype == "bf16"
        K, N, gs = 1024, 2048, 128
        qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=9, sym=False)
        w = oracle.dequant_gptq(qw, qz, sc, None, gs, dtype)
        x = oracle.make_x(M, K, seed=9, dtype=dtype)
        _, want = oracle.gate_up_forward(x, w, oracle_act, None, dtype)
        pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
        # decode sizes run the fused decode kernel; this prefill size splits K (few tiles) and
        # takes the GEMM + elementwise kernel
        got = to_f32(pkg.ops.linear_gate_up(pk, to_dev(x, gpu, bf16=bf), act, fused=True if M == 2 else None))
        assert max_rel_err(got, oracle.to_f32(want, dtype)) <= (TOL_BF16 if bf else TOL)


@pytest.mark.parametrize("K,N,M", [(4096, 28672, 512), (4096, 28672, 2048), (1024, 512, 17), (1024, 768, 300),
                                   (2048, 1024, 129)])
def test_prefill_gate_up(pkg, oracle, gpu, K, N, M):
    assert pkg.ops.select_path(pkg.ops.make_packed(*[to_dev(a, gpu) for a in oracle.make_gptq(K, N, 128, seed=1)[:3]],
                                                   None, 128, 0), M) in ("gemm", "gemv")
    _case(pkg, oracle, gpu, K, N, 128, M, bias=(M == 300), seed=M + 3)


def test_prefill_bf16_groupsize_64(pkg, oracle, gpu):
    _case(pkg, oracle, gpu, 2048, 1024, 64, 640, dtype="bf16", seed=4)


def test_prefill_fused_kernel_where_k_is_not_split(pkg, oracle, gpu):
    """Enough tiles to run unsplit: the MFMA kernel with the gated epilogue; a small grid that
    splits K keeps the two-kernel route and refuses `fused=True`."""
    _case(pkg, oracle, gpu, 1024, 4096, 128, 2048, fused=True, seed=1)
    _case(pkg, oracle, gpu, 1024, 4096, 128, 2048, fused=True, bias=True, act="gelu", seed=2)
    _case(pkg, oracle, gpu, 1024, 4096, 128, 512, fused=True, dtype="bf16", seed=3)
    with pytest.raises(pkg._lib.Q4Error):
        _case(pkg, oracle, gpu, 4096, 512, 128, 128, fused=True, seed=1)


@pytest.mark.parametrize("act", ["silu", "gelu_tanh", "gelu"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K,N,gs,M,bitwise", [(4096, 28672, 128, 2048, True), (4096, 28672, 128, 777, True),
                                              (2048, 8192, 64, 1024, False), (512, 65536, 256, 64, True),
                                              (512, 65536, 128, 33, True)])
def test_prefill_fused_equals_two_kernels_bitwise(pkg, oracle, gpu, act, dtype, K, N, gs, M, bitwise):
    """Same MFMA sequence per column, same roundings, same activation routine: the fused
    epilogue and GEMM + act_mul agree bit for bit (ragged last row tile included).  Where the
    plain GEMM of the two-kernel route runs with two K groups per workgroup (a grid of one
    workgroup per CU) its summation order differs: compared to the parity bar there."""
    bf = dtype == "bf16"
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=M, sym=False)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    x = to_dev(oracle.make_x(M, K, seed=M + 1, dtype=dtype), gpu, bf16=bf)
    rng = np.random.default_rng(M)
    b32 = rng.standard_normal(N).astype(np.float32)
    b = to_dev(b32.astype(np.float16) if not bf else oracle.f32_to_bf16_bits(b32), gpu, bf16=bf)
    for bias in (None, b):
        one = pkg.ops.linear_gate_up(pk, x, act, bias, fused=True)
        two = pkg.ops.linear_gate_up(pk, x, act, bias, fused=False)
        torch.cuda.synchronize()
        if bitwise:
            assert torch.equal(one.view(torch.int16), two.view(torch.int16))
        else:
            assert max_rel_err(to_f32(one), to_f32(two)) <= (TOL_BF16 if bf else TOL)


@pytest.mark.parametrize("layout,act_order", [("awq", False), ("gptq", True)])
@pytest.mark.parametrize("M", [1, 200])
def test_unfused_fallback(pkg, oracle, gpu, layout, act_order, M):
    """AWQ and act-order weights have no fused kernel: linear + elementwise kernel, same result."""
    _case(pkg, oracle, gpu, 2048, 1024, 128, M, layout=layout, act_order=act_order, seed=M + 20)
    with pytest.raises(pkg._lib.Q4Error):
        _case(pkg, oracle, gpu, 2048, 1024, 128, M, layout=layout, act_order=act_order, fused=True, seed=M + 20)


def test_fused_equals_unfused_bitwise_at_decode(pkg, oracle, gpu):
    """Same kernel, same summation order, same roundings: the two routes agree bit for bit."""
    K, N, gs, M = 4096, 28672, 128, 2
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=2)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    x = to_dev(oracle.make_x(M, K, seed=2), gpu)
    a = pkg.ops.linear_gate_up(pk, x, "silu", fused=True)
    b = pkg.ops.linear_gate_up(pk, x, "silu", fused=False)
    # (the unfused route may pick other decode tiles, i.e. another summation order: compare
    # to the parity bar, and bitwise when the orders coincide)
    assert max_rel_err(to_f32(a), to_f32(b)) <= TOL


def test_module_helper(pkg, oracle, gpu):
    K, N, gs, M = 1024, 512, 128, 3
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=6, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, gs, "f16")
    layer = pkg.QuantLinear(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, None, 4, gs)
    x = oracle.make_x(2 * M, K, seed=6).reshape(2, M, K)
    _, want = oracle.gate_up_forward(x.reshape(-1, K), w, "silu", None, "f16")
    got = pkg.gate_up_act(layer, to_dev(x, gpu), "silu")
    assert got.shape == (2, M, N // 2)
    assert max_rel_err(to_f32(got).reshape(-1, N // 2), want.astype(np.float32)) <= TOL


def test_act_mul_kernel_bit_exact(pkg, oracle, gpu):
    """The elementwise kernel against the oracle on its own: silu rounds like the oracle's."""
    rng = np.random.default_rng(0)
    gu = (rng.standard_normal((37, 2 * 264)) * 3).astype(np.float16)
    for act in ("silu", "gelu_tanh", "gelu"):
        a = oracle.activation_f32(gu[:, :264].astype(np.float32), act).astype(np.float16).astype(np.float32)
        want = (a * gu[:, 264:].astype(np.float32)).astype(np.float16)
        got = pkg.ops.act_mul(to_dev(gu, gpu), act).cpu().numpy()
        # tanh / erf of the device library and of NumPy differ in the last fp32 ulp, which the
        # cancellation in 1 + tanh(.) for negative inputs amplifies: a few outputs land on the
        # neighbouring fp16 value
        same = np.mean(got.view(np.uint16) == want.view(np.uint16))
        assert same >= (0.995 if act == "silu" else 0.95), (act, same)
        assert max_rel_err(got.astype(np.float32), want.astype(np.float32)) <= 1e-3
