"""Pins the CPU oracle (oracle/q4_oracle.py) by means other than itself.

No reference code is imported.  The checks are: literal known-answer words, the
reference *writer* algorithm (QuantLinear.pack, triton.py:294-349) restated here with
plain loops and read back by the oracle, element-by-element brute force from the layout
definition, algebraic invariants, and independent implementations of the roundings
(float64 arithmetic, torch's bfloat16 conversion).
"""

import numpy as np
import pytest
import torch

from oracle import q4_oracle as o


# --------------------------------------------------------------------------- literal KATs


def test_unpack_rows_literal():
    # nibble j of a qweight word is row 8r + j (triton.py:160-169: shifter = (k % 8) * 4)
    q = np.array([[0x76543210, 0x00000000], [-19088744, 0x0F0F0F0F]], dtype=np.int64).astype(np.int32)
    assert int(q[1, 0]) & 0xFFFFFFFF == 0xFEDCBA98
    rows = o.unpack_rows(q)
    assert rows.shape == (16, 2)
    assert rows[:8, 0].tolist() == [0, 1, 2, 3, 4, 5, 6, 7]
    assert rows[8:, 0].tolist() == [8, 9, 10, 11, 12, 13, 14, 15]  # sign bit set: 0xFEDCBA98
    assert rows[8:, 1].tolist() == [15, 0, 15, 0, 15, 0, 15, 0]


def test_unpack_cols_literal():
    # nibble j of a qzeros word is column 8c + j (triton.py:167: zeros_shifter = (n % 8) * 4)
    q = np.array([[0x76543210, 0x11111119]], dtype=np.int32)
    cols = o.unpack_cols(q)
    assert cols.tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, 9, 1, 1, 1, 1, 1, 1, 1]]


def test_gptq_zero_plus_one_literal():
    # symmetric checkpoints store 7 in every nibble (0x77777777) and mean zero point 8
    assert (o.gptq_zero_points(np.array([[0x77777777]], dtype=np.int32)) == 8).all()
    # the +1 wraps inside the nibble: 15 -> 0, and never carries into the neighbour
    z = o.gptq_zero_points(np.array([[0x0000F0FF]], dtype=np.int32))
    assert z.tolist() == [[0, 0, 1, 0, 1, 1, 1, 1]]


def test_awq_order_literal():
    assert o.AWQ_PACK_ORDER == [0, 2, 4, 6, 1, 3, 5, 7]  # conversion_utils.py:5
    assert [o.AWQ_PACK_ORDER[o.REVERSE_AWQ_PACK_ORDER[i]] for i in range(8)] == list(range(8))
    assert [o.REVERSE_AWQ_PACK_ORDER[o.AWQ_PACK_ORDER[i]] for i in range(8)] == list(range(8))
    # nibble position p holds logical column ORDER[p]: a word whose nibble p equals p
    # therefore unpacks to column i = value REVERSE[i]
    cols = o.awq_unpack_cols(np.array([[0x76543210]], dtype=np.int32))
    assert cols.tolist() == [[0, 4, 1, 5, 2, 6, 3, 7]]
    # the adjacent-pair property the interleave exists for: nibbles p and p+4 (16 bits apart)
    # are logical neighbours 2p and 2p+1
    for p in range(4):
        assert o.AWQ_PACK_ORDER[p] + 1 == o.AWQ_PACK_ORDER[p + 4]


# --------------------------------------------------------------------------- the reference writer, restated


def reference_style_pack(W, scales_gn, zeros_gn, g_idx):
    """QuantLinear.pack (triton.py:294-349) with explicit loops: returns (qweight, qzeros).

    W [K, N] float32; scales_gn / zeros_gn [G, N]; g_idx [K].  The writer rounds
    (W + zero*scale) / scale to the nibble, packs 8 consecutive K rows per word and stores
    zero - 1 packed 8 columns per word.
    """
    K, N = W.shape
    G = scales_gn.shape[0]
    sz = zeros_gn.astype(np.float32) * scales_gn.astype(np.float32)
    intw = np.zeros((K, N), dtype=np.uint32)
    for k in range(K):
        g = g_idx[k]
        intw[k] = np.round((W[k] + sz[g]) / scales_gn[g].astype(np.float32)).astype(np.int64).astype(np.uint32)
    qweight = np.zeros((K // 8, N), dtype=np.uint32)
    i = 0
    row = 0
    while row < qweight.shape[0]:
        for j in range(i, i + 8):
            qweight[row] |= intw[j] << np.uint32(4 * (j - i))
        i += 8
        row += 1
    zeros = zeros_gn.astype(np.int64) - 1
    zeros = zeros.astype(np.uint32)
    qzeros = np.zeros((G, N // 8), dtype=np.uint32)
    i = 0
    col = 0
    while col < qzeros.shape[1]:
        for j in range(i, i + 8):
            qzeros[:, col] |= (zeros[:, j] & np.uint32(0xF)) << np.uint32(4 * (j - i))
        i += 8
        col += 1
    return qweight.view(np.int32), qzeros.view(np.int32)


@pytest.mark.parametrize("act_order", [False, True])
def test_writer_reader_round_trip(act_order):
    """Weights that are exactly s*(q-z) survive write (reference algorithm) -> read (oracle)."""
    rng = np.random.default_rng(3)
    K, N, gs = 64, 16, 16
    G = K // gs
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(1, 16, size=(G, N))  # the writer stores z-1, so z=0 is not representable
    s = (2.0 ** rng.integers(-8, -3, size=(G, N)) * rng.choice([1.0, 1.5, 1.25], size=(G, N))).astype(np.float16)
    g_idx = np.arange(K) // gs
    if act_order:
        g_idx = g_idx[rng.permutation(K)]
    W = (s[g_idx].astype(np.float32) * (q - z[g_idx]).astype(np.float32))
    assert np.array_equal(W, W.astype(np.float16).astype(np.float32))  # exactly representable
    qweight, qzeros = reference_style_pack(W, s, z, g_idx)
    got = o.dequant_gptq(qweight, qzeros, s, g_idx.astype(np.int32) if act_order else None, gs, "f16")
    assert np.array_equal(got.astype(np.float32), W)
    # and the oracle's own packers agree with the reference-style writer
    assert np.array_equal(o.pack_rows(q), qweight)
    assert np.array_equal(o.pack_cols(z - 1), qzeros)


# --------------------------------------------------------------------------- brute force from the definition


def test_dequant_gptq_brute_force():
    rng = np.random.default_rng(5)
    K, N, gs = 32, 16, 8
    qweight = rng.integers(-(2**31), 2**31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    qzeros = rng.integers(-(2**31), 2**31, size=(K // gs, N // 8), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(1e-3, 2e-2, size=(K // gs, N)).astype(np.float16)
    g_idx = rng.integers(0, K // gs, size=K).astype(np.int32)
    for gi in (None, g_idx):
        got = o.dequant_gptq(qweight, qzeros, scales, gi, gs, "f16")
        for k in range(K):
            for n in range(N):
                word = int(qweight[k >> 3, n]) & 0xFFFFFFFF
                qq = (word >> (4 * (k & 7))) & 0xF
                zword = lambda g: int(qzeros[g, n >> 3]) & 0xFFFFFFFF
                g = int(gi[k]) if gi is not None else k // gs
                zz = (((zword(g) >> (4 * (n & 7))) & 0xF) + 1) & 0xF
                expect = np.float16(np.float64(scales[g, n]) * (qq - zz))  # exact product, one rounding
                assert got[k, n] == expect or (np.isnan(got[k, n]) and np.isnan(expect))


def test_dequant_awq_brute_force():
    rng = np.random.default_rng(6)
    K, N, gs = 16, 16, 8
    qweight = rng.integers(-(2**31), 2**31, size=(K, N // 8), dtype=np.int64).astype(np.int32)
    qzeros = rng.integers(-(2**31), 2**31, size=(K // gs, N // 8), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(1e-3, 2e-2, size=(K // gs, N)).astype(np.float16)
    got = o.dequant_awq(qweight, qzeros, scales, gs, "f16")
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    for k in range(K):
        for c in range(N // 8):
            w = int(qweight[k, c]) & 0xFFFFFFFF
            z = int(qzeros[k // gs, c]) & 0xFFFFFFFF
            for p in range(8):
                n = 8 * c + order[p]
                qq = (w >> (4 * p)) & 0xF
                zz = (z >> (4 * p)) & 0xF  # no +1 in the AWQ format
                assert got[k, n] == np.float16(np.float64(scales[k // gs, n]) * (qq - zz))


# --------------------------------------------------------------------------- invariants


def test_awq_equals_converted_gptq():
    """dequant_awq(q, z, s) == dequant_gptq(fast_awq_to_gptq(q, z), s): the in-tree
    equivalence of awq/conversion_utils.py:83-97."""
    for seed, (K, N, gs) in enumerate([(128, 64, 32), (256, 128, 128), (64, 8, 64)]):
        aq, az, sc = o.make_awq(K, N, gs, seed=seed)
        gq, gz = o.fast_awq_to_gptq(aq, az)
        assert gq.shape == (K // 8, N) and gz.shape == az.shape
        a = o.dequant_awq(aq, az, sc, gs, "f16")
        g = o.dequant_gptq(gq, gz, sc, None, gs, "f16")
        assert np.array_equal(a.view(np.uint16), g.view(np.uint16))


def test_trivial_g_idx_is_no_g_idx():
    qw, qz, sc, _ = o.make_gptq(256, 32, 64, seed=1, sym=False)
    triv = (np.arange(256) // 64).astype(np.int32)
    a = o.dequant_gptq(qw, qz, sc, None, 64)
    b = o.dequant_gptq(qw, qz, sc, triv, 64)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_act_order_row_permutation_invariance():
    """An act-order matrix equals a sequential one whose rows were permuted: row k of the
    act-order W is s[g_idx[k]] * (q[k] - z[g_idx[k]]), so sorting rows by group gives a
    sequential-group matrix, and x @ W is unchanged when x's columns move with the rows
    (what exllama's make_sequential relies on, q_matrix.cu:566-650)."""
    K, N, gs = 128, 16, 32
    qw, qz, sc, g_idx = o.make_gptq(K, N, gs, seed=9, sym=False, act_order=True)
    W = o.dequant_gptq(qw, qz, sc, g_idx, gs)
    perm = np.argsort(g_idx, kind="stable")
    q_sorted = o.unpack_rows(qw)[perm]
    W_seq = o.dequant_gptq(o.pack_rows(q_sorted), qz, sc, None, gs)
    assert np.array_equal(W[perm].view(np.uint16), W_seq.view(np.uint16))
    x = o.make_x(3, K, seed=2)
    y1 = o.matmul_fp32(x.astype(np.float32), W.astype(np.float32))
    y2 = o.matmul_fp32(x[:, perm].astype(np.float32), W_seq.astype(np.float32))
    np.testing.assert_allclose(y1, y2, rtol=1e-5, atol=1e-5)


def test_closed_form_constant_matrix():
    # q = 15 everywhere, stored zero 7 (=8), s = 0.5: W = 3.5; x = ones: y = 3.5 K
    K, N = 64, 8
    qw = o.pack_rows(np.full((K, N), 15))
    qz = o.pack_cols(np.full((1, N), 7))
    sc = np.full((1, N), 0.5, dtype=np.float16)
    W = o.dequant_gptq(qw, qz, sc, None, K)
    assert (W == np.float16(3.5)).all()
    y32, y16 = o.linear_forward(np.ones((2, K), dtype=np.float16), W, None, "f16")
    assert (y32 == 3.5 * K).all() and (y16 == np.float16(3.5 * K)).all()


def test_pack_unpack_round_trips():
    rng = np.random.default_rng(0)
    m = rng.integers(0, 16, size=(32, 24), dtype=np.uint8)
    assert np.array_equal(o.unpack_rows(o.pack_rows(m)), m)
    assert np.array_equal(o.unpack_cols(o.pack_cols(m)), m)
    assert np.array_equal(o.awq_unpack_cols(o.awq_pack_cols(m)), m)


# --------------------------------------------------------------------------- roundings and matmul


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    a = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 10.0 ** rng.integers(-6, 6, 4096).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40, -1e-40], dtype=np.float32),
    ])
    ours = o.f32_to_bf16_bits(a)
    ref = torch.from_numpy(a).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, ref)
    assert np.array_equal(o.bf16_bits_to_f32(ours), torch.from_numpy(a).to(torch.bfloat16).float().numpy())


def test_dequant_bf16_is_single_rounding():
    qw, qz, sc, _ = o.make_gptq(128, 32, 32, seed=4, sym=False)
    got = o.dequant_gptq(qw, qz, sc, None, 32, "bf16")
    q = o.unpack_rows(qw).astype(np.float64)
    z = o.gptq_zero_points(qz).astype(np.float64)
    g = np.arange(128) // 32
    exact = sc[g].astype(np.float64) * (q - z[g])
    ref = torch.from_numpy(exact).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, ref)


def test_matmul_against_float64_and_identity():
    qw, qz, sc, _ = o.make_gptq(256, 64, 128, seed=2, sym=False)
    W = o.dequant_gptq(qw, qz, sc, None, 128)
    x = o.make_x(5, 256, seed=3)
    y32, y16 = o.linear_forward(x, W, None, "f16")
    y64 = x.astype(np.float64) @ W.astype(np.float64)
    assert np.abs(y32 - y64).max() <= 1e-5 * np.abs(y64).max()
    assert np.array_equal(y16, y32.astype(np.float16))
    eye = np.eye(256, dtype=np.float16)
    w_back, _ = o.linear_forward(eye, W, None, "f16")
    assert np.array_equal(w_back, W.astype(np.float32))
    # leading dims and bias follow the module contract (triton.py:351-363)
    x3 = x.reshape(5, 1, 256)
    b = np.arange(64, dtype=np.float16)
    y3, y3c = o.linear_forward(x3, W, b, "f16")
    assert y3.shape == (5, 1, 64)
    np.testing.assert_allclose(y3[:, 0], y32 + b.astype(np.float32), rtol=0, atol=0)
    assert np.array_equal(y3c[:, 0], (y16.astype(np.float32) + b.astype(np.float32)).astype(np.float16))


def test_synthetic_generators_match_config():
    qw, qz, sc, gi = o.make_gptq(256, 64, 128, seed=0, sym=True, act_order=True)
    assert qw.shape == (32, 64) and qw.dtype == np.int32
    assert (qz.view(np.uint32) == 0x77777777).all()
    assert sc.dtype == np.float16 and sc.min() >= np.float16(1e-3) and sc.max() <= np.float16(2e-2)
    assert sorted(np.bincount(gi).tolist()) == [128, 128]  # every group has exactly 128 rows
    q = o.unpack_rows(qw)
    assert q.min() == 0 and q.max() == 15


def test_activations_known_values(oracle):
    """Closed forms: silu(0) = 0, silu(x) + silu(-x) = x; gelu(x) - gelu(-x) = x for both
    variants; large |x| limits; a dropped factor or sign fails one of them."""
    x = np.linspace(-6, 6, 97, dtype=np.float32)
    for act in ("silu", "gelu", "gelu_tanh"):
        a = oracle.activation_f32(x, act)
        assert a[48] == 0.0
        assert np.allclose(a - oracle.activation_f32(-x, act), x, atol=2e-6)
        assert abs(a[-1] - 6.0) < 2e-2 and abs(a[0]) < 2e-2
    assert np.isclose(oracle.activation_f32(np.float32([1.0]), "silu")[0], 1.0 / (1.0 + np.exp(-1.0)), rtol=1e-6)
    assert np.isclose(oracle.activation_f32(np.float32([1.0]), "gelu")[0], 0.8413447460685429, rtol=1e-6)
    assert np.isclose(oracle.activation_f32(np.float32([1.0]), "gelu_tanh")[0], 0.8411919906082768, rtol=1e-6)


def test_gate_up_forward_roundings(oracle):
    """act(gate) * up on a hand-made case: every intermediate is rounded to fp16."""
    w = np.zeros((2, 4), dtype=np.float16)
    w[0, 0] = 1.0      # gate_0 = x_0
    w[1, 1] = 1.0      # gate_1 = x_1
    w[0, 2] = 3.0      # up_0 = 3 x_0
    w[1, 3] = 0.5      # up_1 = x_1 / 2
    x = np.array([[1.0, -2.0]], dtype=np.float16)
    exact, out = oracle.gate_up_forward(x, w, "silu")
    s1 = np.float16(1.0 / (1.0 + np.exp(-1.0)))
    s2 = np.float16(-2.0 / (1.0 + np.exp(2.0)))
    assert out.dtype == np.float16 and out.shape == (1, 2)
    assert out[0, 0] == np.float16(np.float32(s1) * np.float32(3.0))
    assert out[0, 1] == np.float16(np.float32(s2) * np.float32(-1.0))
    assert np.allclose(exact[0], [3.0 / (1.0 + np.exp(-1.0)), 2.0 / (1.0 + np.exp(2.0))], rtol=1e-6)


def test_torch_restatement_matches_numpy_oracle():
    """The PyTorch restatement used for the CPU baseline is the NumPy oracle in another idiom:
    same dequantized bits, same fp32 products (GPTQ with and without g_idx, AWQ)."""
    import torch

    from oracle import q4_oracle as o
    from oracle import q4_oracle_torch as ot

    def t(a):
        return torch.from_numpy(a.view(np.int32) if a.dtype == np.uint32 else a)

    for act in (False, True):
        qw, qz, sc, gi = o.make_gptq(512, 256, 128, seed=7, sym=False, act_order=act)
        w = o.dequant_gptq(qw, qz, sc, gi, 128, "f16")
        wt = ot.dequant_gptq(t(qw), t(qz), t(sc), t(gi) if gi is not None else None, 128)
        assert np.array_equal(wt.numpy().view(np.uint16), w.view(np.uint16))
    qw, qz, sc = o.make_awq(512, 256, 128, seed=8)
    w = o.dequant_awq(qw, qz, sc, 128, "f16")
    wt = ot.dequant_awq(t(qw), t(qz), t(sc), 128)
    assert np.array_equal(wt.numpy().view(np.uint16), w.view(np.uint16))
    x = o.make_x(5, 512, seed=3)
    y32, y16 = o.linear_forward(x, w, None, "f16")
    t32, t16 = ot.linear_forward(t(x), wt, None)
    assert np.allclose(t32.numpy(), y32, rtol=1e-5, atol=1e-5)
    assert np.array_equal(wt.numpy()[:1].view(np.uint16), w[:1].view(np.uint16))
    # one-hot rows read the weights back exactly through the matmul
    eye = torch.eye(512, dtype=torch.float16)[:7]
    assert torch.equal(ot.linear_forward(eye, wt, None)[1], wt[:7])
