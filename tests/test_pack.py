"""QuantLinear.pack: the offline writer of the GPTQ layout (reference: gptq/triton.py:294-349).

The writer is checked against what the layout fixes, not against itself: a matrix built as
s*(q - z) must come back as exactly the nibbles q and the zero points z - 1 when the packed
tensors are read by the oracle's independent unpackers, and the dequantized matrix must be
the original one bit for bit.  A brute-force loop over single elements pins the rounding
rule (half to even, division by the fp16 scale) on weights that do not sit on the grid.
"""

from __future__ import annotations

from types import SimpleNamespace

import numpy as np
import pytest
import torch


def dense_layer(W, bias=None):
    """Stand-in for the nn.Linear the reference's writer takes: weight is [N, K]."""
    return SimpleNamespace(weight=torch.from_numpy(np.ascontiguousarray(W.T)), bias=bias)


def grid_case(rng, K, N, gs, act_order):
    G = K // gs
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(1, 17, size=(G, N))  # the writer stores z - 1
    s = (2.0 ** rng.integers(-8, -3, size=(G, N)) * rng.choice([1.0, 1.5, 1.25], size=(G, N))).astype(np.float16)
    g_idx = np.arange(K) // gs
    if act_order:
        g_idx = g_idx[rng.permutation(K)]
    W = s[g_idx].astype(np.float32) * (q - z[g_idx]).astype(np.float32)
    return q, z, s, g_idx.astype(np.int32), W


@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("K,N,gs", [(64, 16, 16), (256, 64, 128), (128, 8, 32)])
def test_pack_round_trip(pkg, oracle, K, N, gs, act_order):
    rng = np.random.default_rng(K + N + act_order)
    q, z, s, g_idx, W = grid_case(rng, K, N, gs, act_order)
    layer = pkg.QuantLinear.new(4, gs, K, N, bias=False)
    layer.pack(
        dense_layer(W),
        torch.from_numpy(s.T.astype(np.float32).copy()),
        torch.from_numpy(z.T.astype(np.float32).copy()),
        torch.from_numpy(g_idx) if act_order else None,
    )
    qweight = layer.qweight.numpy()
    qzeros = layer.qzeros.numpy()
    assert qweight.dtype == np.int32 and qweight.shape == (K // 8, N)
    assert qzeros.dtype == np.int32 and qzeros.shape == (K // gs, N // 8)
    assert layer.scales.dtype == torch.float16 and tuple(layer.scales.shape) == (K // gs, N)
    assert np.array_equal(oracle.unpack_rows(qweight), q)
    assert np.array_equal(oracle.unpack_cols(qzeros), (z - 1) & 15)
    assert np.array_equal(oracle.gptq_zero_points(qzeros), z & 15)
    assert np.array_equal(layer.scales.numpy(), s)
    got = oracle.dequant_gptq(qweight, qzeros, s, g_idx if act_order else None, gs, "f16")
    if (z < 16).all():
        assert np.array_equal(got.astype(np.float32), W)
    else:  # zero 16 is stored as 15 and read back as 0: the format cannot hold it
        keep = (z < 16)[g_idx]
        assert np.array_equal(got.astype(np.float32)[keep], W[keep])


def test_pack_rounding_rule_brute_force(pkg, oracle):
    """Off-grid weights: every nibble is round_half_even((w + z*s) / fp16(s)) in fp32."""
    rng = np.random.default_rng(11)
    K, N, gs = 32, 8, 16
    G = K // gs
    s32 = rng.uniform(0.01, 0.05, size=(G, N)).astype(np.float32)
    z = rng.integers(1, 16, size=(G, N)).astype(np.float32)
    target = rng.uniform(0.0, 15.0, size=(K, N)).astype(np.float32)
    target[0, :] = np.arange(N) + 0.5  # ties
    g = np.arange(K) // gs
    s16 = s32.astype(np.float16)
    W = (target * s16[g].astype(np.float32) - z[g] * s32[g]).astype(np.float32)
    layer = pkg.QuantLinear.new(4, gs, K, N, bias=False)
    layer.pack(dense_layer(W), torch.from_numpy(s32.T.copy()), torch.from_numpy(z.T.copy()))
    got = oracle.unpack_rows(layer.qweight.numpy())
    for k in range(K):
        for n in range(N):
            num = np.float32(W[k, n]) + np.float32(z[g[k], n]) * np.float32(s32[g[k], n])
            val = np.float32(num) / np.float32(s16[g[k], n])
            want = int(np.rint(val))  # rint rounds half to even
            assert 0 <= want <= 15
            assert got[k, n] == want, (k, n, val)


def test_pack_keeps_bias_and_drops_stale_kernel_view(pkg):
    rng = np.random.default_rng(2)
    K, N, gs = 64, 16, 32
    q, z, s, g_idx, W = grid_case(rng, K, N, gs, False)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32))
    layer = pkg.QuantLinear.new(4, gs, K, N, bias=True)
    layer._packed = object()
    layer.pack(dense_layer(W, bias), torch.from_numpy(s.T.astype(np.float32).copy()), torch.from_numpy(z.T.astype(np.float32).copy()))
    assert layer._packed is None
    assert layer.bias.dtype == torch.float16
    assert torch.equal(layer.bias, bias.half())
    # the caller's tensors are left alone
    assert torch.equal(bias, bias.clone())


def test_pack_zero_point_zero_wraps_like_the_reference(pkg):
    """zero 0 is stored as -1: every bit from its nibble upwards is set in that word."""
    K, N, gs = 32, 8, 32
    s = np.full((1, N), 0.5, dtype=np.float32)
    z = np.full((1, N), 8.0, dtype=np.float32)
    z[0, 2] = 0.0
    W = np.zeros((K, N), dtype=np.float32)
    layer = pkg.QuantLinear.new(4, gs, K, N, bias=False)
    layer.pack(dense_layer(W), torch.from_numpy(s.T.copy()), torch.from_numpy(z.T.copy()))
    word = int(layer.qzeros.numpy().view(np.uint32)[0, 0])
    assert word == (0x77777777 | (0xFFFFFFFF << 8)) & 0xFFFFFFFF
