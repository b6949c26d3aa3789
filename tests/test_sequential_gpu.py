"""Act-order by row order: q4_gptq_make_sequential + q4_gather_columns (exllamav2's
make_sequential / q_perm, q_matrix.cu:524-640) against the oracle.

The repacked matrix is pinned by what the layout fixes: unpacking its rows with the oracle's
independent unpacker must give exactly the checkpoint rows in perm order, the dequantized matrix
handed back in checkpoint order must equal the oracle's act-order dequantization bit for bit,
and the forward must agree with the oracle like every other path (and with the table-lookup
kernels, which take the same weights in checkpoint order)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 2e-3


def to_dev(a, gpu):
    if a is None:
        return None
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu)


def max_rel_err(got, ref):
    return float(np.abs(got - ref).max() / max(1e-6, np.abs(ref).max()))


def build(pkg, oracle, gpu, K, N, gs, seed):
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=seed, sym=False, act_order=True)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    return qw, qz, sc, gi, pk


@pytest.mark.parametrize("K,N,gs", [(256, 64, 32), (1024, 512, 128), (4096, 1024, 128), (512, 264, 64)])
def test_rows_are_the_checkpoint_rows_in_group_order(pkg, oracle, gpu, K, N, gs):
    qw, qz, sc, gi, pk = build(pkg, oracle, gpu, K, N, gs, seed=K + N)
    seq = pkg.ops.make_sequential(pk)
    assert seq is not None and seq.g_idx is None and seq.perm.dtype == torch.int32
    perm = seq.perm.cpu().numpy()
    assert sorted(perm.tolist()) == list(range(K))
    assert np.array_equal(gi[perm], np.arange(K) // gs)          # group order
    assert all(np.all(np.diff(perm[g * gs:(g + 1) * gs]) > 0) for g in range(K // gs))  # stable
    rows = oracle.unpack_rows(qw)
    got = oracle.unpack_rows(seq.qweight.cpu().numpy())
    assert np.array_equal(got, rows[perm])
    # dequantized and handed back in checkpoint order: the act-order matrix, bit for bit
    want = oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16")
    w = pkg.ops.dequantize(seq)
    assert np.array_equal(w.cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("M", [1, 3, 16, 40, 300])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_forward_matches_oracle_and_table_kernels(pkg, oracle, gpu, M, dtype):
    K, N, gs = 2048, 1024, 128
    qw, qz, sc, gi, pk = build(pkg, oracle, gpu, K, N, gs, seed=M)
    seq = pkg.ops.make_sequential(pk)
    bf = dtype == "bf16"
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype)
    xh = oracle.make_x(M, K, seed=M + 1, dtype=dtype)
    x = torch.from_numpy(xh.view(np.int16)).to(gpu).view(torch.bfloat16) if bf else to_dev(xh, gpu)
    y32, _ = oracle.linear_forward(xh, w, None, dtype)
    got = pkg.ops.linear(seq, x)
    g = got.float().cpu().numpy()
    assert max_rel_err(g, y32) <= (8e-3 if bf else TOL)
    if not bf:  # the table-lookup decode kernel is fp16 only
        ref = pkg.ops.linear(pk, x).float().cpu().numpy()
        assert max_rel_err(g, ref) <= TOL


@pytest.mark.parametrize("path,M", [(1, 2), (1, 18), (1, 40), (2, 40), (2, 700), (3, 5)])
def test_forced_paths_read_x_through_perm(pkg, oracle, gpu, path, M):
    """Decode kernels gather while staging (one, two and several row blocks), the prefill and
    generic paths gather into the workspace tail first: same result as gathering by hand."""
    K, N, gs = 4096, 512, 128
    qw, qz, sc, gi, pk = build(pkg, oracle, gpu, K, N, gs, seed=path * 100 + M)
    seq = pkg.ops.make_sequential(pk)
    x = to_dev(oracle.make_x(M, K, seed=M), gpu)
    bias = to_dev(np.random.default_rng(M).standard_normal(N).astype(np.float16), gpu)
    got = pkg.ops.linear(seq, x, bias, path=path)
    plain = pkg.ops.PackedWeight(seq.qweight, seq.qzeros, seq.scales, None, K, N, gs, K // gs, 0)
    want = pkg.ops.linear(plain, x[:, seq.perm.long()].contiguous(), bias, path=path)
    if path == 1 and M <= 3:
        # up to three rows the plain call runs the short-launch kernel, the call through perm the
        # kernel that gathers while it stages: same sums, roundings of different arithmetic
        assert float((got.float() - want.float()).abs().max() / want.float().abs().max()) <= 2e-3
    else:
        assert torch.equal(got, want)
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16")
    y32, _ = oracle.linear_forward(x.cpu().numpy(), w, bias.cpu().numpy(), "f16")
    assert max_rel_err(got.float().cpu().numpy(), y32) <= TOL


def test_prefill_with_perm_needs_the_larger_workspace(pkg, oracle, gpu):
    import ctypes
    K, N, gs, M = 1024, 256, 128, 64
    qw, qz, sc, gi, pk = build(pkg, oracle, gpu, K, N, gs, seed=2)
    seq = pkg.ops.make_sequential(pk)
    lib = pkg._lib.load()
    small = int(lib.q4_workspace_bytes(M, K, N))
    assert int(lib.q4_workspace_bytes_perm(M, K, N)) >= small + M * K * 2
    ws = torch.zeros(small, dtype=torch.uint8, device=gpu)
    x = torch.zeros((M, K), dtype=torch.float16, device=gpu)
    y = torch.zeros((M, N), dtype=torch.float16, device=gpu)
    st = seq.struct()
    rc = lib.q4_linear_perm(ctypes.byref(st), seq.perm.data_ptr(), x.data_ptr(), None, y.data_ptr(), M, 0,
                            ws.data_ptr(), ws.numel(), 2, None)
    assert rc == pkg._lib.ERR_WORKSPACE
    assert b"q4_workspace_bytes_perm" in lib.q4_last_error()


def test_gather_columns_is_exact(pkg, gpu):
    g = torch.Generator(device=gpu).manual_seed(3)
    x = torch.randn((37, 1024), device=gpu, dtype=torch.float16, generator=g)
    perm = torch.randperm(1024, device=gpu, generator=g).to(torch.int32)
    assert torch.equal(pkg.ops.gather_columns(x, perm), x[:, perm.long()])
    xb = x.to(torch.bfloat16)
    assert torch.equal(pkg.ops.gather_columns(xb, perm), xb[:, perm.long()])
    # many rows: the kernel that stages each row in LDS; K = 40000 does not fit and falls back
    big = torch.randn((300, 1024), device=gpu, dtype=torch.float16, generator=g)
    assert torch.equal(pkg.ops.gather_columns(big, perm), big[:, perm.long()])
    wide = torch.randn((130, 40000), device=gpu, dtype=torch.float16, generator=g)
    pw = torch.randperm(40000, device=gpu, generator=g).to(torch.int32)
    assert torch.equal(pkg.ops.gather_columns(wide, pw), wide[:, pw.long()])


def test_groups_of_unequal_size_are_left_alone(pkg, oracle, gpu):
    """A g_idx whose groups do not all hold `groupsize` rows cannot become contiguous."""
    K, N, gs = 512, 64, 128
    qw, qz, sc, gi, _ = build(pkg, oracle, gpu, K, N, gs, seed=1)
    gi = gi.copy()
    gi[np.flatnonzero(gi == 1)[0]] = 0  # group 0 gets 129 rows
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    assert pkg.ops.make_sequential(pk) is None


def test_argument_validation(pkg, gpu):
    lib = pkg._lib.load()
    L = pkg._lib
    t = torch.zeros(64, dtype=torch.int32, device=gpu)
    assert lib.q4_gptq_make_sequential(None, t.data_ptr(), t.data_ptr(), 64, 8, None) == L.ERR_INVALID_ARGUMENT
    assert lib.q4_gptq_make_sequential(t.data_ptr(), t.data_ptr(), t.data_ptr(), 64, 8, None) == L.ERR_INVALID_ARGUMENT
    o = torch.zeros(64, dtype=torch.int32, device=gpu)
    assert lib.q4_gptq_make_sequential(t.data_ptr(), t.data_ptr(), o.data_ptr(), 60, 8, None) == L.ERR_INVALID_ARGUMENT
    assert lib.q4_gather_columns(t.data_ptr(), t.data_ptr(), o.data_ptr(), 1, 12, None) == L.ERR_UNSUPPORTED
    assert lib.q4_gather_columns(t.data_ptr(), t.data_ptr(), o.data_ptr(), 0, 12, None) == 0


def _act_order_mode(monkeypatch, mode):
    import importlib
    mod = importlib.import_module("text-generation-inference_amd.layers.gptq.quant_linear")
    monkeypatch.setattr(mod, "ACT_ORDER_MODE", mode)


@pytest.mark.parametrize("mode", ["table", "repack"])
@pytest.mark.parametrize("cls", ["triton", "exllama"])
def test_act_order_modules_leave_the_checkpoint_tensors_alone(pkg, oracle, gpu, monkeypatch, mode, cls):
    """Both act-order routes of the modules: the default reads the checkpoint layout through
    g_idx; Q4_ACT_ORDER=repack keeps a private copy with the rows in group order.  Either way
    the tensors the loader handed in (and with them the state_dict) are never written."""
    _act_order_mode(monkeypatch, mode)
    K, N, gs = 1024, 256, 128
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=5, sym=False, act_order=True)
    tq, tz, ts, tg = to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu)
    if cls == "triton":
        layer = pkg.QuantLinear(tq, tz, ts, tg, None, 4, gs)
        pk = layer.packed()
    else:
        weight = pkg.GPTQWeight(qweight=tq, qzeros=tz, scales=ts, g_idx=tg, bits=4, groupsize=gs,
                                use_awq_kernel=False, use_exllama=True)
        layer = pkg.get_linear(weight, None)
        pk = layer._packed
    assert (pk.perm is not None) == (mode == "repack") and (pk.g_idx is not None) == (mode == "table")
    xh = oracle.make_x(4, K, seed=9)
    x = to_dev(xh, gpu)
    y1 = layer(x)
    y2 = layer(x)
    assert torch.equal(y1, y2)
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16")
    y32, _ = oracle.linear_forward(xh, w, None, "f16")
    assert max_rel_err(y1.float().cpu().numpy(), y32) <= TOL
    assert np.array_equal(layer.dequantize().cpu().numpy().view(np.uint16), w.view(np.uint16))
    # the loader's tensors are what they were
    assert np.array_equal(tq.cpu().numpy().view(np.uint32), qw.view(np.uint32)) and np.array_equal(tg.cpu().numpy(), gi)
    if cls == "triton":
        assert layer.qweight.data_ptr() == tq.data_ptr() and layer.g_idx.data_ptr() == tg.data_ptr()
        sd = layer.state_dict()
        assert np.array_equal(sd["qweight"].cpu().numpy().view(np.uint32), qw.view(np.uint32)) and np.array_equal(sd["g_idx"].cpu().numpy(), gi)
        # a copy of the module (new storage) rebuilds its kernel view and keeps working
        import copy
        twin = copy.deepcopy(layer)
        assert torch.equal(twin(x), y1)
    else:
        assert layer.q_tensors.qweight.data_ptr() == tq.data_ptr()


@pytest.mark.parametrize("M", [1, 16, 200])
def test_wqlinear_both_routes_agree_and_keep_the_checkpoint_layout(pkg, oracle, gpu, M, monkeypatch):
    """The AWQ module reads its checkpoint layout directly by default; Q4_AWQ=convert serves a
    private GPTQ-layout copy: same dense matrix bit for bit (zero point 0 included: stored 15,
    read back as 0), same outputs to rounding, and `qweight` keeps its [K, N/8] shape."""
    K, N, gs = 1024, 512, 128
    aq, az, sc = oracle.make_awq(K, N, gs, seed=M)
    az = az.copy()
    az[0, :4] = 0  # whole words of zero points 0
    want = oracle.dequant_awq(aq, az, sc, gs, "f16")
    import importlib
    mod = importlib.import_module("text-generation-inference_amd.layers.awq.quantize")
    monkeypatch.setattr(mod, "AWQ_MODE", "convert")
    conv = pkg.WQLinear(4, gs, to_dev(aq, gpu), to_dev(az, gpu), to_dev(sc, gpu), None)
    xh = oracle.make_x(M, K, seed=M + 2)
    x = to_dev(xh, gpu)
    y = conv(x)
    assert tuple(conv.qweight.shape) == (K, N // 8) and conv.packed().layout == 0
    assert np.array_equal(conv.qweight.cpu().numpy().view(np.uint32), aq.view(np.uint32))
    assert np.array_equal(conv.dequantize().cpu().numpy().view(np.uint16), want.view(np.uint16))
    y32, _ = oracle.linear_forward(xh, want, None, "f16")
    assert max_rel_err(y.float().cpu().numpy(), y32) <= TOL
    monkeypatch.setattr(mod, "AWQ_MODE", "native")
    native = pkg.WQLinear(4, gs, to_dev(aq, gpu), to_dev(az, gpu), to_dev(sc, gpu), None)
    yn = native(x)
    assert native.packed().layout == 1 and native.packed().qweight.data_ptr() == native.qweight.data_ptr()
    assert np.array_equal(native.dequantize().cpu().numpy().view(np.uint16), want.view(np.uint16))
    assert max_rel_err(yn.float().cpu().numpy(), y32) <= TOL
    assert max_rel_err(y.float().cpu().numpy(), yn.float().cpu().numpy()) <= TOL


def test_out_of_range_permutation_entries_are_clamped(pkg, oracle, gpu):
    """A permutation with entries outside 0..K-1 must not read outside x or qweight: such entries
    are clamped to the nearest valid index in the repack kernel, the gather kernels and the
    decode kernel's fused gather."""
    K, N, gs = 1024, 256, 128
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=4, sym=False)
    qd = to_dev(qw, gpu)
    bad = torch.arange(K, dtype=torch.int32, device=gpu)
    bad[3] = -7
    bad[100] = K + 12345
    bad[1023] = 2**31 - 1
    clamped = bad.clamp(0, K - 1)
    lib = pkg._lib.load()
    out_bad, out_ok = torch.empty_like(qd), torch.empty_like(qd)
    assert lib.q4_gptq_make_sequential(qd.data_ptr(), bad.data_ptr(), out_bad.data_ptr(), K, N, None) == 0
    assert lib.q4_gptq_make_sequential(qd.data_ptr(), clamped.data_ptr(), out_ok.data_ptr(), K, N, None) == 0
    assert torch.equal(out_bad, out_ok)
    x = to_dev(oracle.make_x(2, K, seed=1), gpu)
    assert torch.equal(pkg.ops.gather_columns(x, bad), x[:, clamped.long()])
    plain = pkg.ops.make_packed(qd, to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    with_bad = pkg.ops.PackedWeight(plain.qweight, plain.qzeros, plain.scales, None, K, N, gs, K // gs, 0, bad)
    with_ok = pkg.ops.PackedWeight(plain.qweight, plain.qzeros, plain.scales, None, K, N, gs, K // gs, 0, clamped)
    for M in (1, 2, 5, 40):  # fused gather (1, 2 rows), workspace gather, prefill
        xm = to_dev(oracle.make_x(M, K, seed=M), gpu)
        assert torch.equal(pkg.ops.linear(with_bad, xm), pkg.ops.linear(with_ok, xm))


@pytest.mark.parametrize("K,M", [(2048, 1), (2048, 2), (8192, 1), (2048, 5), (2048, 300)])
def test_gated_mlp_first_half_on_rows_in_group_order(pkg, oracle, gpu, K, M):
    """act(gate) * up with a [gate | up] weight in group order: the fused decode kernel gathers
    while staging (K <= 4096) or after a gather pass (longer K); more rows take linear + act_mul.
    All agree with the same computation on hand-gathered activations and with the oracle."""
    N, gs = 512, 128
    qw, qz, sc, gi, pk = build(pkg, oracle, gpu, K, N, gs, seed=K // 256 + M)
    seq = pkg.ops.make_sequential(pk)
    xh = oracle.make_x(M, K, seed=M + 11)
    x = to_dev(xh, gpu)
    got = pkg.ops.linear_gate_up(seq, x, "silu")
    plain = pkg.ops.PackedWeight(seq.qweight, seq.qzeros, seq.scales, None, K, N, gs, K // gs, 0)
    want = pkg.ops.linear_gate_up(plain, x[:, seq.perm.long()].contiguous(), "silu")
    assert torch.equal(got, want)
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16")
    _, ref = oracle.gate_up_forward(xh, w, "silu", None, "f16")
    assert max_rel_err(got.float().cpu().numpy(), oracle.to_f32(ref, "f16")) <= TOL


@pytest.mark.parametrize("gate_up_act_order", [False, True])
def test_down_permutation_folded_into_gate_up_columns(pkg, oracle, gpu, gate_up_act_order, monkeypatch):
    """The gated MLP of an act-order model: applying the down projection's permutation to the
    gate and up output columns at load time leaves every output as it was with the run-time gather
    (bit for bit where both routes run the same kernel), and the down projection becomes a plain
    contiguous-group layer."""
    _act_order_mode(monkeypatch, "repack")
    H, I, gs = 1024, 2048, 128
    gq = oracle.make_gptq(H, 2 * I, gs, seed=1, sym=False, act_order=gate_up_act_order)
    dq = oracle.make_gptq(I, H, gs, seed=2, sym=False, act_order=True)
    rng = np.random.default_rng(0)
    bias = to_dev(rng.standard_normal(2 * I).astype(np.float16), gpu)

    def layers():
        gu = pkg.QuantLinear(to_dev(gq[0], gpu), to_dev(gq[1], gpu), to_dev(gq[2], gpu),
                             to_dev(gq[3], gpu) if gq[3] is not None else
                             (torch.arange(H, device=gpu) // gs).to(torch.int32), bias.clone(), 4, gs)
        dn = pkg.QuantLinear(to_dev(dq[0], gpu), to_dev(dq[1], gpu), to_dev(dq[2], gpu), to_dev(dq[3], gpu), None, 4, gs)
        return gu, dn

    gu0, dn0 = layers()
    gu1, dn1 = layers()
    assert pkg.fold_down_permutation(gu1, dn1)
    assert dn1.packed().perm is None and dn0.packed().perm is not None
    assert not pkg.fold_down_permutation(gu1, dn1)  # nothing left to fold
    for M in (1, 3, 16, 100):
        x = to_dev(oracle.make_x(M, H, seed=M), gpu)
        y0 = dn0(pkg.gate_up_act(gu0, x, "silu"))
        y1 = dn1(pkg.gate_up_act(gu1, x, "silu"))
        if M <= 3:
            # up to three rows the folded (plain) down projection runs the short-launch kernel, the
            # one that still gathers the kernel that gathers while it stages: different roundings
            assert float((y0.float() - y1.float()).abs().max() / y0.float().abs().max()) <= 2e-3, M
        else:
            assert torch.equal(y0, y1), M
    # against the oracle, once
    wg = oracle.dequant_gptq(gq[0], gq[1], gq[2], gq[3], gs, "f16")
    wd = oracle.dequant_gptq(dq[0], dq[1], dq[2], dq[3], gs, "f16")
    xh = oracle.make_x(4, H, seed=9)
    _, h = oracle.gate_up_forward(xh, wg, "silu", bias.cpu().numpy(), "f16")
    y32, _ = oracle.linear_forward(h, wd, None, "f16")
    got = dn1(pkg.gate_up_act(gu1, to_dev(xh, gpu), "silu")).float().cpu().numpy()
    assert max_rel_err(got, y32) <= 2 * TOL
