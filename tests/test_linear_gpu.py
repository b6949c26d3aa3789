"""GPU parity of y = x @ dequant(W): every kernel path against the oracle.

Bar (BASELINE.json north_star): max|y - ref| / max|ref| <= 2e-3 against an
fp32-accumulated reference built from the bit-exact dequantized weights.  The fp16/bf16
output rounding itself is up to 2^-11 / 2^-8 relative, so the comparison target is the
oracle's output rounded to the activation dtype; the fp32 value is checked too.
"""

import numpy as np
import pytest
import torch

from tests.util import max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu

TOL = 2e-3       # north_star tolerance, fp16
TOL_BF16 = 8e-3  # bf16 output rounding alone is 2^-8 = 3.9e-3 per element


def _run(pkg, oracle, gpu, K, N, gs, M, dtype="f16", layout="gptq", sym=True, act=False, bias=False, path=0, cfg=None, seed=0):
    bf = dtype == "bf16"
    if layout == "gptq":
        qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=seed, sym=sym, act_order=act)
        w = oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype)
        lay = 0
    else:
        qw, qz, sc = oracle.make_awq(K, N, gs, seed=seed)
        gi = None
        w = oracle.dequant_awq(qw, qz, sc, gs, dtype)
        lay = 1
    x = oracle.make_x(M, K, seed=seed, dtype=dtype)
    b = None
    if bias:
        rng = np.random.default_rng(seed + 1)
        bf32 = rng.standard_normal(N).astype(np.float32)
        b = bf32.astype(np.float16) if not bf else oracle.f32_to_bf16_bits(bf32)
    y32, ycast = oracle.linear_forward(x, w, b, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, lay)
    xt = to_dev(x, gpu, bf16=bf)
    bt = to_dev(b, gpu, bf16=bf)
    got = pkg.ops.linear(pk, xt, bt, path=path, gemv_config=cfg)
    torch.cuda.synchronize()
    assert got.shape == (M, N)
    assert got.dtype == (torch.bfloat16 if bf else torch.float16)
    g = to_f32(got)
    assert np.isfinite(g).all()
    err = max_rel_err(g, y32)
    assert err <= (TOL_BF16 if bf else TOL), f"max rel err {err:.3e}"
    return g, y32


GEMV_SHAPES = [(4096, 4096), (4096, 6144), (4096, 28672), (14336, 4096)]


def test_cfg1_gptq_m16(pkg, oracle, gpu):
    """BASELINE.json configs[0]: K=N=4096, groupsize 128, sym, M=16."""
    _run(pkg, oracle, gpu, 4096, 4096, 128, 16, seed=1)


@pytest.mark.parametrize("K,N", GEMV_SHAPES)
@pytest.mark.parametrize("M", [1, 2, 4, 8, 16])
def test_gemv_llama3_8b(pkg, oracle, gpu, K, N, M):
    pk_path = 1  # force the decode kernel
    _run(pkg, oracle, gpu, K, N, 128, M, path=pk_path, seed=K // 64 + N // 64 + M)


@pytest.mark.parametrize("M", [1, 3, 5, 7, 11, 13, 16])
def test_gemv_ragged_m_asym_bias(pkg, oracle, gpu, M):
    _run(pkg, oracle, gpu, 1024, 512, 128, M, sym=False, bias=True, path=1, seed=M)


@pytest.mark.parametrize("gs", [32, 64, 128, 256, 512, -1])
def test_gemv_groupsizes(pkg, oracle, gpu, gs):
    _run(pkg, oracle, gpu, 1024, 256, gs, 3, sym=False, path=1, seed=gs + 100)


@pytest.mark.parametrize("cfg", [(1, 1, 1), (1, 1, 8), (2, 1, 4), (4, 1, 2), (1, 4, 2), (2, 2, 2), (4, 2, 1), (1, 8, 1), (2, 4, 1), (4, 1, 16)])
@pytest.mark.parametrize("M", [1, 6, 16])
def test_gemv_decompositions(pkg, oracle, gpu, cfg, M):
    _run(pkg, oracle, gpu, 2048, 1024, 128, M, sym=False, bias=(M == 6), cfg=cfg, seed=sum(cfg) + M)


def test_gemv_config_that_exceeds_lds_is_refused(pkg, oracle, gpu):
    """16 rows x 14336 K values do not fit the 160 KB of LDS in one split: the library must
    refuse the decomposition with a clear error instead of launching."""
    with pytest.raises(pkg._lib.Q4Error, match="LDS"):
        _run(pkg, oracle, gpu, 14336, 256, 128, 16, cfg=(1, 1, 1), seed=1)


def test_gemv_bf16(pkg, oracle, gpu):
    _run(pkg, oracle, gpu, 4096, 4096, 128, 8, dtype="bf16", sym=False, path=1, seed=9)


def test_gemv_deterministic_and_tickets_reset(pkg, oracle, gpu):
    """Split-K combines partials in a fixed order: repeated calls are bit-identical, and
    the ticket counters return to zero so the same workspace serves the next call."""
    a, _ = _run(pkg, oracle, gpu, 4096, 4096, 128, 4, path=1, seed=3)
    b, _ = _run(pkg, oracle, gpu, 4096, 4096, 128, 4, path=1, seed=3)
    assert np.array_equal(a, b)
    for ws in pkg.ops._workspaces.values():
        assert int(ws[: pkg._lib.WORKSPACE_COUNTER_BYTES].sum().item()) == 0


@pytest.mark.parametrize("K,N", [(4096, 4096), (14336, 4096), (4096, 6144), (8192, 1024)])
def test_gemv_single_row_fixed_point_combine(pkg, oracle, gpu, K, N):
    """M = 1, fp16: the K splits meet in 64-bit fixed-point cells (integer adds, so the sum does
    not depend on arrival order).  Bit-reproducible, cells back at zero, and the same row
    computed through the ticket path (the row repeated to M = 4) agrees to fp16 rounding."""
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=K + N, sym=False)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    x = to_dev(oracle.make_x(1, K, seed=5), gpu)
    a = pkg.ops.linear(pk, x, None, path=1)
    b = pkg.ops.linear(pk, x, None, path=1)
    two = pkg.ops.linear(pk, torch.cat([x, x, x, x]), None, path=1)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    for ws in pkg.ops._workspaces.values():
        assert int(ws[: pkg._lib.WORKSPACE_COUNTER_BYTES].sum().item()) == 0
    w = oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")
    y32, _ = oracle.linear_forward(x.cpu().numpy(), w, None, "f16")
    assert max_rel_err(to_f32(a), y32) <= TOL
    assert max_rel_err(to_f32(a), to_f32(two[:1])) <= 1e-3
    assert float((a == two[:1]).float().mean()) > 0.9


@pytest.mark.parametrize("layout,act", [("gptq", False), ("gptq", True), ("awq", False)])
@pytest.mark.parametrize("M", [2, 3])
def test_gemv_few_rows_fixed_point_combine(pkg, oracle, gpu, layout, act, M):
    """Two and three fp16 rows also meet in the cells, a row at a time, each wave's sums
    transposed so that one atomic instruction covers 64 consecutive cells.  Same checks as for
    one row; the ticket path (the rows padded to M = 4) is the second opinion."""
    K, N = 4096, 4096
    if layout == "awq":
        qw, qz, sc = oracle.make_awq(K, N, 128, seed=M)
        gi = None
        w = oracle.dequant_awq(qw, qz, sc, 128, "f16")
    else:
        qw, qz, sc, gi = oracle.make_gptq(K, N, 128, seed=M, sym=False, act_order=act)
        w = oracle.dequant_gptq(qw, qz, sc, gi, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), 128,
                             1 if layout == "awq" else 0)
    xh = oracle.make_x(M, K, seed=7 + M)
    x = to_dev(xh, gpu)
    bias = to_dev(np.random.default_rng(M).standard_normal(N).astype(np.float16), gpu)
    a = pkg.ops.linear(pk, x, bias, path=1).clone()
    b = pkg.ops.linear(pk, x, bias, path=1).clone()
    pad = torch.cat([x, x[: 4 - M]])
    four = pkg.ops.linear(pk, pad, bias, path=1)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    for ws in pkg.ops._workspaces.values():
        assert int(ws[: pkg._lib.WORKSPACE_COUNTER_BYTES].sum().item()) == 0
    y32, _ = oracle.linear_forward(xh, w, bias.cpu().numpy(), "f16")
    assert max_rel_err(to_f32(a), y32) <= TOL
    assert max_rel_err(to_f32(a), to_f32(four[:M])) <= 1e-3
    assert float((a == four[:M]).float().mean()) > 0.9


@pytest.mark.parametrize("gs", [32, 64, 128, -1])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("M", [17, 20])
def test_gemv_two_row_blocks(pkg, oracle, gpu, M, dtype, gs):
    """17..20 rows on the contiguous-group decode kernel: one workgroup runs two MFMA row blocks
    per unpacked word (rows 16.. are the second block; its dead rows stay out of the output)."""
    _run(pkg, oracle, gpu, 2048, 512, gs, M, dtype=dtype, sym=False, bias=(M == 20), path=1, seed=M + 3)


@pytest.mark.parametrize("K,N", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_gemv_two_row_blocks_llama_shapes(pkg, oracle, gpu, K, N):
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=1)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    assert pkg.ops.select_path(pk, 18) == "gemv"
    _run(pkg, oracle, gpu, K, N, 128, 18, sym=False, seed=K // 128 + 18)


def test_gemv_single_row_non_finite_input_leaves_the_cells_clean(pkg, oracle, gpu):
    """inf / NaN activations in different K splits make every output non-finite (as in the
    reference; opposite infinities must not cancel) and must not leave anything behind in the
    accumulation cells: the next call is exact again."""
    K, N = 4096, 4096
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=3, sym=False)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    good = to_dev(oracle.make_x(1, K, seed=8), gpu)
    want = pkg.ops.linear(pk, good, None, path=1).clone()
    bad = good.clone()
    bad[0, 5] = float("inf")
    bad[0, 4000] = float("nan")
    y = pkg.ops.linear(pk, bad, None, path=1)
    torch.cuda.synchronize()
    assert not bool(torch.isfinite(y).any())
    for ws in pkg.ops._workspaces.values():
        assert int(ws[: pkg._lib.WORKSPACE_COUNTER_BYTES].sum().item()) == 0
    assert torch.equal(pkg.ops.linear(pk, good, None, path=1), want)


@pytest.mark.parametrize("layout,act", [("gptq", True), ("awq", False), ("gptq", False)])
@pytest.mark.parametrize("M", [1, 5, 33])
def test_generic_path(pkg, oracle, gpu, layout, act, M):
    _run(pkg, oracle, gpu, 1000 if layout == "gptq" and not act else 1024, 264, 40 if (layout == "gptq" and not act) else 128, M,
         layout=layout, sym=False, act=act, bias=True, path=3, seed=M + 50)


# --------------------------------------------------------------------------- prefill GEMM


@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 6144), (14336, 4096)])
@pytest.mark.parametrize("M", [512, 2048])
def test_gemm_llama3_8b_fp16(pkg, oracle, gpu, K, N, M):
    _run(pkg, oracle, gpu, K, N, 128, M, path=2, seed=K // 128 + N // 128 + M)


def test_gemm_gate_up_bf16(pkg, oracle, gpu):
    """BASELINE.json configs[2]: bf16 activations, widest projection."""
    _run(pkg, oracle, gpu, 4096, 28672, 128, 512, dtype="bf16", path=2, seed=77)


@pytest.mark.parametrize("M", [17, 64, 100, 129, 300])
def test_gemm_ragged_m_asym_bias(pkg, oracle, gpu, M):
    _run(pkg, oracle, gpu, 1024, 512, 128, M, sym=False, bias=True, path=2, seed=M)


@pytest.mark.parametrize("gs", [32, 64, 128, 256, -1])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_groupsizes(pkg, oracle, gpu, gs, dtype):
    _run(pkg, oracle, gpu, 1024, 256, gs, 96, dtype=dtype, sym=False, path=2, seed=gs + 200)


@pytest.mark.parametrize("gs", [32, 64])
@pytest.mark.parametrize("dtype,M", [("f16", 2048), ("bf16", 1000), ("f16", 300)])
def test_gemm_two_k_groups_small_groupsizes(pkg, oracle, gpu, gs, dtype, M):
    """A grid of at most 256 tiles of 128 x 256: two K groups of four waves per workgroup (128 rows
    of K per round), with two and four quantisation groups to a round; M = 300 adds split-K."""
    _run(pkg, oracle, gpu, 512, 4096, gs, M, dtype=dtype, sym=False, bias=True, path=2, seed=gs + M)


@pytest.mark.parametrize("K,N,M,gs,dtype,bias", [(256, 6144, 2048, 128, "f16", False), (512, 6144, 1999, 64, "bf16", True),
                                                  (256, 6144, 1536, 256, "f16", True), (192, 3072, 4096, 64, "f16", False),
                                                  (320, 6144, 1290, -1, "bf16", False)])
def test_gemm_wide_tile(pkg, oracle, gpu, K, N, M, gs, dtype, bias):
    """N a multiple of 384 and a grid of 257 .. 511 tiles of 128 x 256: the launch takes the
    128 x 384 tile of eight 48-column waves (gemm_gptq_wide_kernel).  Full and ragged last row
    tiles, an odd number of K tiles, group sizes, asymmetric zero points, bias, both dtypes."""
    _run(pkg, oracle, gpu, K, N, gs, M, dtype=dtype, sym=False, bias=bias, path=2, seed=K + M)


def test_gemm_wide_tile_bit_exact_weights(pkg, oracle, gpu):
    """One-hot activation rows through the 128 x 384 tile: row m of the output is row k(m) of the
    dequantized matrix bit for bit (column order of the three fragments, the 96-bit word loads
    and the paired stores of the epilogue included)."""
    K, N, gs, M = 256, 6144, 128, 2048
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=12, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    ks = np.arange(M) % K
    x = torch.zeros((M, K), dtype=torch.float16, device=gpu)
    x[torch.arange(M, device=gpu), torch.from_numpy(ks).to(gpu)] = 1.0
    got = pkg.ops.linear(pk, x, None, path=2)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), w[ks].view(np.uint16))


def test_gemm_bit_exact_weights_through_identity(pkg, oracle, gpu):
    """x = identity rows: y[m, :] must be W[m, :] exactly (fp16 W is what the MFMA sees, and
    a one-hot fp32 accumulation adds nothing), so the in-register unpack of the GEMM kernel is
    pinned bit for bit against the oracle's dequantized matrix."""
    K, N, gs = 512, 256, 128
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=11, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    eye = torch.eye(K, dtype=torch.float16, device=gpu)
    got = pkg.ops.linear(pk, eye, None, path=2)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), w.view(np.uint16))


@pytest.mark.parametrize("K,N,M,dtype", [(4096, 4096, 512, "f16"), (14336, 4096, 300, "f16"), (4096, 6144, 129, "bf16"),
                                         (1024, 512, 100, "f16"), (2048, 1280, 64, "f16"), (4096, 1024, 1000, "bf16")])
def test_gemm_split_k(pkg, oracle, gpu, K, N, M, dtype):
    """Few output tiles: the K loop is split over workgroups, fp32 partial tiles meet in the
    reduction kernel (fixed split order: bit-reproducible), bias and rounding happen there."""
    a, _ = _run(pkg, oracle, gpu, K, N, 128, M, dtype=dtype, sym=False, bias=True, path=2, seed=K // 64 + N // 64 + M)
    b, _ = _run(pkg, oracle, gpu, K, N, 128, M, dtype=dtype, sym=False, bias=True, path=2, seed=K // 64 + N // 64 + M)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("layout,act", [("awq", False), ("gptq", True)])
@pytest.mark.parametrize("K,N,M", [(4096, 512, 200), (14336, 1024, 96), (2048, 4096, 130)])
def test_gemm_split_k_awq_and_act_order(pkg, oracle, gpu, layout, act, K, N, M):
    a, _ = _run(pkg, oracle, gpu, K, N, 128, M, layout=layout, act=act, sym=False, bias=True, path=2, seed=K // 64 + N + M)
    b, _ = _run(pkg, oracle, gpu, K, N, 128, M, layout=layout, act=act, sym=False, bias=True, path=2, seed=K // 64 + N + M)
    assert np.array_equal(a, b)


def test_gemm_without_workspace_runs_unsplit(pkg, oracle, gpu):
    """No workspace -> one workgroup per whole tile; same result to the parity bar."""
    import ctypes

    K, N, M, gs = 4096, 1024, 300, 128
    qw, qz, sc, _ = oracle.make_gptq(K, N, gs, seed=5, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, gs, "f16")
    x = oracle.make_x(M, K, seed=5)
    y32, _ = oracle.linear_forward(x, w, None, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 0)
    xt = to_dev(x, gpu)
    y = torch.empty((M, N), dtype=torch.float16, device=gpu)
    st = pk.struct()
    rc = pkg._lib.load().q4_linear_ex(ctypes.byref(st), xt.data_ptr(), None, y.data_ptr(), M, 0, None, 0, 2,
                                      torch.cuda.current_stream().cuda_stream)
    pkg._lib.check(rc)
    torch.cuda.synchronize()
    assert max_rel_err(to_f32(y), y32) <= TOL
    assert max_rel_err(to_f32(pkg.ops.linear(pk, xt, None, path=2)), y32) <= TOL


def test_auto_dispatch(pkg, oracle, gpu):
    """q4_linear picks decode for M <= 16 and the MFMA GEMM above, generic for odd shapes."""
    qw, qz, sc, _ = oracle.make_gptq(1024, 512, 128, seed=3)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    assert pkg.ops.select_path(pk, 1) == "gemv"
    assert pkg.ops.select_path(pk, 16) == "gemv"
    assert pkg.ops.select_path(pk, 64) == "gemv"   # small matrix: row-blocked decode up to 64 rows
    assert pkg.ops.select_path(pk, 65) == "gemm"
    qw, qz, sc, _ = oracle.make_gptq(1000, 264, 40, seed=3)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 40, 0)
    assert pkg.ops.select_path(pk, 1) == "generic"
    assert pkg.ops.select_path(pk, 2048) == "generic"


# --------------------------------------------------------------------------- AWQ and act-order decode kernels


@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
@pytest.mark.parametrize("M", [1, 2, 4, 16])
def test_awq_decode_mistral(pkg, oracle, gpu, K, N, M):
    """BASELINE.json configs[4]: AWQ GEMM layout, asymmetric zeros, Mistral-7B shapes, decode kernel."""
    _run(pkg, oracle, gpu, K, N, 128, M, layout="awq", path=1, seed=K // 256 + M)


@pytest.mark.parametrize("M", [3, 7, 16, 17, 40, 64, 256])
def test_awq_m_sweep_chunked(pkg, oracle, gpu, M):
    """The AWQ decode kernel takes any M in row chunks of 16 (BASELINE.json configs[4] sweeps M up to 256);
    so does whatever the dispatch picks for that M."""
    _run(pkg, oracle, gpu, 1024, 512, 128, M, layout="awq", bias=(M % 2 == 1), path=1, seed=M)
    _run(pkg, oracle, gpu, 1024, 512, 128, M, layout="awq", bias=(M % 2 == 1), seed=M)


@pytest.mark.parametrize("gs", [32, 64, 128, 256, -1])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_awq_groupsizes_dtypes(pkg, oracle, gpu, gs, dtype):
    _run(pkg, oracle, gpu, 512, 256, gs, 5, dtype=dtype, layout="awq", path=1, seed=gs + 7)


@pytest.mark.parametrize("cfg", [(1, 1, 1), (1, 4, 2), (2, 2, 1), (1, 8, 1), (2, 1, 4)])
def test_awq_decompositions(pkg, oracle, gpu, cfg):
    _run(pkg, oracle, gpu, 1024, 512, 128, 6, layout="awq", cfg=cfg, seed=sum(cfg))


def test_awq_auto_path_is_native(pkg, oracle, gpu):
    qw, qz, sc = oracle.make_awq(1024, 512, 128, seed=0)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 1)
    for M in (1, 4, 6):
        assert pkg.ops.select_path(pk, M) == "gemv"
    for M in (7, 9, 17, 100, 256):
        assert pkg.ops.select_path(pk, M) == "gemm"  # the register-unpack MFMA kernel, split-K on small grids
    qw, qz, sc, gi = oracle.make_gptq(1024, 512, 128, seed=0, act_order=True)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), 128, 0)
    # two 16-row blocks of the decode kernel still beat the MFMA kernel
    assert pkg.ops.select_path(pk, 32) == "gemv" and pkg.ops.select_path(pk, 33) == "gemm"
    # too many groups for an LDS parameter table: the gathering kernel pays off later
    qw, qz, sc, gi = oracle.make_gptq(8192, 128, 32, seed=0, act_order=True)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), 32, 0)
    assert pkg.ops.select_path(pk, 48) == "gemv" and pkg.ops.select_path(pk, 49) == "gemm"


@pytest.mark.parametrize("K,N", [(8192, 10240), (28672, 8192)])
@pytest.mark.parametrize("M", [1, 16])
def test_act_order_decode_llama70b(pkg, oracle, gpu, K, N, M):
    """BASELINE.json configs[3]: desc_act=True with a random row permutation, Llama-3-70B per-layer shapes."""
    _run(pkg, oracle, gpu, K, N, 128, M, act=True, path=1, seed=K // 1024 + M)


@pytest.mark.parametrize("K,N,M", [(4096, 14336, 1), (4096, 14336, 8), (4096, 28672, 16), (14336, 4096, 16),
                                   (18944, 3584, 1), (3584, 4608, 1), (3584, 4608, 16), (4096, 22016, 2)])
def test_act_order_decode_picker_branches(pkg, oracle, gpu, K, N, M):
    """The lookup kernels' picker: two column tiles per workgroup on wide layers, the single
    round of workgroups it takes with 12 rows or more when the slab leaves one workgroup per CU,
    a split count held to one round of workgroups (18944 rows), four K waves on a short K that
    does not deal out over eight (3584 rows), and a second round taken lightly at one or two rows."""
    _run(pkg, oracle, gpu, K, N, 128, M, act=True, sym=False, path=1, seed=N // 1024 + M)


@pytest.mark.parametrize("K,gs", [(14336, 32), (17920, 32), (28672, 64)])
@pytest.mark.parametrize("M,dtype", [(1, "f16"), (16, "f16"), (3, "bf16")])
def test_act_order_decode_many_groups(pkg, oracle, gpu, K, gs, M, dtype):
    """448 and 560 groups: the parameter table of a 64-column tile takes 112 / 140 KB of LDS and
    the decode kernel still runs, beside a g_idx slice of a K range split far enough."""
    N = 512
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=3, act_order=True)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    assert pkg.ops.select_path(pk, M) == "gemv"
    _run(pkg, oracle, gpu, K, N, gs, M, dtype=dtype, act=True, sym=False, path=1, seed=K // 512 + M)


@pytest.mark.parametrize("M", [1, 5, 16, 33, 128])
def test_act_order_small(pkg, oracle, gpu, M):
    _run(pkg, oracle, gpu, 1024, 256, 128, M, sym=False, act=True, bias=True, seed=M + 300)


@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("cfg", [(1, 1, 1), (1, 4, 2), (2, 2, 2), (1, 8, 1)])
def test_act_order_groupsizes_decompositions(pkg, oracle, gpu, gs, cfg):
    _run(pkg, oracle, gpu, 2048, 256, gs, 4, sym=False, act=True, cfg=cfg, seed=gs + sum(cfg))


def test_act_order_bit_exact_weights_through_identity(pkg, oracle, gpu):
    """One-hot activations read the unpacked act-order weights back exactly."""
    K, N, gs = 256, 128, 32
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=21, sym=False, act_order=True)
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    eye = torch.eye(K, dtype=torch.float16, device=gpu)
    got = pkg.ops.linear(pk, eye, None, path=1)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), w.view(np.uint16))


def test_gptq_decode_m_chunks(pkg, oracle, gpu):
    """The GPTQ decode kernel also runs M > 16 in row chunks when forced."""
    _run(pkg, oracle, gpu, 1024, 512, 128, 50, sym=False, bias=True, path=1, seed=50)


@pytest.mark.parametrize("cfg", [(1, 8, 1, 1), (1, 4, 2, 1), (2, 4, 1, 2), (1, 8, 1, 2), (4, 2, 1, 1), (1, 1, 4, 2)])
@pytest.mark.parametrize("M", [1, 2, 7, 16])
def test_gemv_narrow_column_tiles(pkg, oracle, gpu, cfg, M):
    """16- and 32-column tiles per wave (1 or 2 packed words per lane) of the GPTQ decode kernel."""
    _run(pkg, oracle, gpu, 1024, 512, 128, M, sym=False, bias=(M == 7), cfg=cfg, seed=sum(cfg) + M)


@pytest.mark.parametrize("gs", [256, -1])
def test_gemv_narrow_tiles_large_groups(pkg, oracle, gpu, gs):
    _run(pkg, oracle, gpu, 1024, 256, gs, 3, sym=False, cfg=(1, 4, 1, 1), seed=gs + 1)


# --------------------------------------------------------------------------- AWQ prefill GEMM


@pytest.mark.parametrize("K,N,M", [(4096, 14336, 256), (14336, 4096, 512), (1024, 512, 130)])
def test_awq_gemm(pkg, oracle, gpu, K, N, M):
    """AWQ layout through the MFMA kernel that unpacks the weight tile into LDS."""
    _run(pkg, oracle, gpu, K, N, 128, M, layout="awq", path=2, bias=(M == 130), seed=K // 512 + M)


@pytest.mark.parametrize("gs", [32, 64, 128, -1])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_awq_gemm_groupsizes_dtypes(pkg, oracle, gpu, gs, dtype):
    _run(pkg, oracle, gpu, 512, 256, gs, 100, dtype=dtype, layout="awq", path=2, seed=gs + 11)


def test_awq_gemm_bit_exact_weights_through_identity(pkg, oracle, gpu):
    K, N, gs = 512, 256, 128
    qw, qz, sc = oracle.make_awq(K, N, gs, seed=31)
    w = oracle.dequant_awq(qw, qz, sc, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, gs, 1)
    eye = torch.eye(K, dtype=torch.float16, device=gpu)
    got = pkg.ops.linear(pk, eye, None, path=2)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), w.view(np.uint16))


def test_awq_dispatch_large_m(pkg, oracle, gpu):
    qw, qz, sc = oracle.make_awq(1024, 14336, 128, seed=0)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 1)
    assert pkg.ops.select_path(pk, 6) == "gemv"
    assert pkg.ops.select_path(pk, 7) == "gemm"
    assert pkg.ops.select_path(pk, 64) == "gemm"
    # the kernel that unpacks the words in registers (groups of 64 rows or more, N a multiple of
    # 256) takes over from 7 rows on whatever the shape
    for K, N in [(4096, 4096), (4096, 6144), (14336, 4096), (4096, 14336), (8192, 28672), (28672, 8192)]:
        w = pkg.ops.PackedWeight(pk.qweight, pk.qzeros, pk.scales, None, K, N, 128, K // 128, 1)  # geometry only
        assert pkg.ops.select_path(w, 6) == "gemv", (K, N)
        assert pkg.ops.select_path(w, 7) == "gemm", (K, N)
    # groups of 32 rows go through the kernel that unpacks through LDS: the first row count that
    # goes to it moves with the shape (measured crossovers)
    for K, N, first in [(4096, 4096, 9), (4096, 6144, 14), (11008, 4096, 10), (14336, 4096, 17), (4096, 14336, 17),
                        (8192, 10240, 17), (8192, 28672, 33), (28672, 8192, 33)]:
        w = pkg.ops.PackedWeight(pk.qweight, pk.qzeros, pk.scales, None, K, N, 32, K // 32, 1)  # geometry only
        assert pkg.ops.select_path(w, first - 1) == "gemv", (K, N)
        assert pkg.ops.select_path(w, first) == "gemm", (K, N)


def test_gemm_n_multiple_of_128_only(pkg, oracle, gpu):
    """N = 384 is not a multiple of 256: the GEMM takes its 128-column tile."""
    _run(pkg, oracle, gpu, 1024, 384, 128, 3000, sym=False, bias=True, path=2, seed=384)


# --------------------------------------------------------------------------- K that does not divide evenly


@pytest.mark.parametrize("layout,act", [("gptq", False), ("gptq", True), ("awq", False)])
@pytest.mark.parametrize("M", [1, 3, 16, 20])
def test_gemv_ragged_k_partition(pkg, oracle, gpu, layout, act, M):
    """K = 43 chunks of 128 rows (prime): the wave slots get two or three chunks each
    (Llama-2-7B's down projection has K = 11008 = 86 chunks)."""
    _run(pkg, oracle, gpu, 43 * 128, 512, 128, M, layout=layout, act=act, sym=False, bias=(M == 3), path=1, seed=M + 43)


@pytest.mark.parametrize("cfg", [(1, 4, 3), (1, 4, 5), (2, 2, 7), (1, 8, 2), (1, 3, 5), (1, 1, 43)])
def test_gemv_ragged_k_explicit_decompositions(pkg, oracle, gpu, cfg):
    """43 chunks over wk x splits slots that do not divide them."""
    _run(pkg, oracle, gpu, 43 * 128, 256, 128, 5, sym=False, cfg=cfg, seed=sum(cfg))
    _run(pkg, oracle, gpu, 43 * 128, 256, 64, 2, sym=False, cfg=cfg, seed=sum(cfg) + 1)


@pytest.mark.parametrize("layout,act", [("gptq", False), ("gptq", True), ("awq", False)])
def test_decode_picker_sweep(pkg, oracle, gpu, layout, act):
    """Whatever decomposition the picker chooses must be launchable and right: chunk counts
    with awkward divisors, narrow and wide N, every row count of a block and beyond."""
    rng = np.random.default_rng(7)
    cases = []
    for chunks in (1, 2, 3, 5, 7, 9, 11, 13, 24, 43):
        for N in ((256, 512) if layout == "awq" else (64, 192, 512)):
            cases.append((chunks * 128, N, int(rng.integers(1, 21))))
    cases += [(86 * 128, 1024, 16), (40 * 128, 2048, 12), (108 * 128, 768 if layout != "awq" else 1024, 5)]
    for K, N, M in cases:
        _run(pkg, oracle, gpu, K, N, 128, M, layout=layout, act=act, sym=False, path=1, seed=K // 128 + N + M)


def test_gemv_llama2_7b_down_shape(pkg, oracle, gpu):
    _run(pkg, oracle, gpu, 11008, 4096, 128, 1, path=1, seed=11)
    _run(pkg, oracle, gpu, 11008, 4096, 128, 16, path=1, seed=12)


def test_gemv_rejects_more_wave_slots_than_chunks(pkg, oracle, gpu):
    with pytest.raises(pkg._lib.Q4Error):
        _run(pkg, oracle, gpu, 512, 256, 128, 2, cfg=(1, 4, 2))  # 4 chunks, 8 slots


# --------------------------------------------------------------------------- act-order prefill GEMM


@pytest.mark.parametrize("K,N,M", [(8192, 10240, 1024), (1024, 256, 200), (2048, 128, 64)])
def test_act_order_gemm(pkg, oracle, gpu, K, N, M):
    """BASELINE.json configs[3], prefill: desc_act through the MFMA kernel (per-row scale/zero gathered by g_idx)."""
    _run(pkg, oracle, gpu, K, N, 128, M, sym=(K == 8192), act=True, path=2, bias=(M == 200), seed=K // 512 + M)


@pytest.mark.parametrize("gs", [32, 128])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_act_order_gemm_groupsizes_dtypes(pkg, oracle, gpu, gs, dtype):
    _run(pkg, oracle, gpu, 512, 256, gs, 70, dtype=dtype, sym=False, act=True, path=2, seed=gs + 13)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("K,gs,N,M", [(2048, 128, 256, 100),      # 16 groups: 32-bit LDS table
                                       (6400, 32, 256, 100),       # 200 groups: scale + zero-byte LDS table
                                       (8192, 32, 128, 100),       # 256 groups: per-row global gather
                                       (4096, 128, 11008, 300)])   # 258 tiles: the table that lets two share a CU
def test_act_order_gemm_parameter_sources(pkg, oracle, gpu, K, gs, N, M, dtype):
    """Every way the act-order MFMA kernel fetches a row's scale and zero point."""
    _run(pkg, oracle, gpu, K, N, gs, M, dtype=dtype, sym=False, act=True, path=2, bias=True, seed=K // 64 + gs)


@pytest.mark.parametrize("K,gs", [(512, 64), (6400, 32), (8192, 32)])
def test_act_order_gemm_bit_exact_weights_through_identity(pkg, oracle, gpu, K, gs):
    N = 128
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=33, sym=False, act_order=True)
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    eye = torch.eye(K, dtype=torch.float16, device=gpu)
    got = pkg.ops.linear(pk, eye, None, path=2)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), w.view(np.uint16))


def test_act_order_gemm_out_of_range_group_index_is_clamped(pkg, oracle, gpu):
    """A corrupt g_idx must not send the kernel outside its table: entries are clamped to
    the first and last group, as in the dequantize kernel."""
    K, N, gs = 1024, 128, 128
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=4, sym=False, act_order=True)
    bad = gi.copy()
    bad[5] = 1000
    bad[77] = -3
    clamped = gi.copy()
    clamped[5] = K // gs - 1
    clamped[77] = 0
    w = oracle.dequant_gptq(qw, qz, sc, clamped, gs, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(bad, gpu), gs, 0)
    eye = torch.eye(K, dtype=torch.float16, device=gpu)
    got = pkg.ops.linear(pk, eye, None, path=2)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), w.view(np.uint16))


def test_act_order_dispatch(pkg, oracle, gpu):
    qw, qz, sc, gi = oracle.make_gptq(1024, 10240, 128, seed=0, act_order=True)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), 128, 0)
    assert pkg.ops.select_path(pk, 16) == "gemv"
    assert pkg.ops.select_path(pk, 1024) == "gemm"
    assert pkg.ops.select_path(pk, 1024, torch.bfloat16) == "gemm"
    assert pkg.ops.select_path(pk, 4, torch.bfloat16) == "gemv"


@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("K,N", [(1024, 1024), (8192, 10240)])
def test_act_order_bf16_small_m(pkg, oracle, gpu, K, N, M):
    """g_idx with bf16 activations at decode sizes: the lookup decode kernel with bf16 weights
    rounded once from the fp32 product, and the MFMA kernel forced on the same problem."""
    _run(pkg, oracle, gpu, K, N, 128, M, dtype="bf16", act=True, seed=M + 2)
    _run(pkg, oracle, gpu, K, N, 128, M, dtype="bf16", act=True, seed=M + 2, path=2)


@pytest.mark.parametrize("zeros", ["random", "one", "one_but_a_column"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_act_order_decode_one_hot_reads_weights_back(pkg, oracle, gpu, dtype, zeros):
    """x = rows of the identity through the lookup decode kernel: the dequantized rows, bit for bit.
    The kernel takes a shorter loop when every zero point of a workgroup's 64 columns is the same
    (symmetric quantization): random zero points, one zero point everywhere, and one zero point
    except in a single (group, column) - whose column tile must take the general loop while its
    neighbours take the short one."""
    K, N, gs = 1024, 512, 128
    bf = dtype == "bf16"
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=11, sym=(zeros != "random"), act_order=True)
    if zeros == "one_but_a_column":
        qz = qz.copy()
        qz[5, 200 // 8] ^= np.int32(0x3 << (4 * (200 % 8)))  # group 5, column 200: stored zero 7 -> 4
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    ks = np.random.default_rng(2).choice(K, size=8, replace=False)
    x = torch.zeros((8, K), dtype=torch.bfloat16 if bf else torch.float16, device=gpu)
    for i, k in enumerate(ks):
        x[i, k] = 1.0
    y = pkg.ops.linear(pk, x, None, path=1)
    torch.cuda.synchronize()
    got = y.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, w[ks].view(np.uint16))


# --------------------------------------------------------------------------- full-size properties


@pytest.mark.parametrize("K,N", [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)])
def test_llama3_8b_shapes_size_independent_properties(pkg, oracle, gpu, K, N):
    """At the benchmark's full sizes, properties that need no CPU matmul: one-hot activations read
    single weight rows back bit for bit through every decode combine (cells for 1..3 rows, tickets,
    two row blocks) and through the prefill GEMM; the decode and prefill kernels agree on random
    activations; y is linear in x to rounding."""
    g = torch.Generator(device=gpu).manual_seed(K + N)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K // 8, N), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    qzeros = torch.randint(-(2**31), 2**31 - 1, (K // 128, N // 8), dtype=torch.int64, device=gpu, generator=g).to(torch.int32)
    scales = (torch.rand((K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    w = pkg.ops.make_packed(qweight, qzeros, scales, None, 128, 0)
    dense = pkg.ops.dequantize(w)  # bit-exact against the oracle in the dequant tests
    rows = torch.randint(0, K, (40,), device=gpu, generator=g)
    for M in (1, 3, 8, 18, 40):
        x = torch.zeros((M, K), dtype=torch.float16, device=gpu)
        x[torch.arange(M, device=gpu), rows[:M]] = 1.0
        y = pkg.ops.linear(w, x)
        assert torch.equal(y, dense[rows[:M]]), f"one-hot rows, M={M}"
    x = torch.zeros((40, K), dtype=torch.float16, device=gpu)
    x[torch.arange(40, device=gpu), rows] = 1.0
    assert torch.equal(pkg.ops.linear(w, x, path=2), dense[rows])
    a = torch.randn((16, K), device=gpu, dtype=torch.float16, generator=g)
    b = torch.randn((16, K), device=gpu, dtype=torch.float16, generator=g)
    ya, yb = pkg.ops.linear(w, a, path=1).float(), pkg.ops.linear(w, b, path=1).float()
    ga = pkg.ops.linear(w, a, path=2).float()
    scale = float(ya.abs().max())
    assert float((ya - ga).abs().max()) <= 2e-3 * scale          # decode against prefill kernel
    yab = pkg.ops.linear(w, (a.float() * 0.5 + b.float() * 0.5).half(), path=1).float()
    assert float((yab - 0.5 * (ya + yb)).abs().max()) <= 4e-3 * scale  # linearity to input/output rounding


@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("poison", ["+inf", "-inf", "nan", "+inf,-inf"])
def test_decode_non_finite_activations_keep_their_class(pkg, oracle, gpu, M, poison):
    """inf / NaN activations through split-K (accumulation cells up to 3 rows, tickets from 4):
    every output is NaN, +inf or -inf exactly where fp32 arithmetic on the dequantized weights
    gives that class, and the rows without poison stay finite and correct."""
    K, N = 4096, 4096
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=77, sym=False)
    w = oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    x = oracle.make_x(M, K, seed=M).copy()
    vals = {"+inf": np.inf, "-inf": -np.inf, "nan": np.nan}
    for i, name in enumerate(poison.split(",")):
        x[M - 1, 100 + 1500 * i] = np.float16(vals[name])
    with np.errstate(invalid="ignore", over="ignore"):
        ref = x.astype(np.float32) @ w.astype(np.float32)
    got = to_f32(pkg.ops.linear(pk, to_dev(x, gpu), None, path=1))
    torch.cuda.synchronize()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isposinf(got), np.isposinf(ref))
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    fin = np.isfinite(ref)
    if fin.any():
        assert np.abs(got[fin] - ref[fin]).max() <= TOL * np.abs(ref[fin]).max()
    # a later clean call finds the cells and tickets as the kernels must leave them
    xc = oracle.make_x(M, K, seed=M + 40)
    clean = to_f32(pkg.ops.linear(pk, to_dev(xc, gpu), None, path=1))
    assert np.isfinite(clean).all()
    assert max_rel_err(clean, xc.astype(np.float32) @ w.astype(np.float32)) <= TOL


@pytest.mark.parametrize("layout", ["gptq", "awq"])
def test_decode_offset_kernels_stay_non_finite_on_poisoned_rows(pkg, oracle, gpu, layout):
    """The kernels that keep the splice offsets in the sums (large GPTQ layers, AWQ up to 8 rows)
    subtract inf from inf on a poisoned row: its outputs are non-finite (NaN where the reference
    may say +-inf); other rows are untouched."""
    K, N, M = 4096, 14336, 2
    if layout == "gptq":
        qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=5)
        w = oracle.dequant_gptq(qw, qz, sc, None, 128, "f16")
    else:
        qw, qz, sc = oracle.make_awq(K, N, 128, seed=5)
        w = oracle.dequant_awq(qw, qz, sc, 128, "f16")
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0 if layout == "gptq" else 1)
    x = oracle.make_x(M, K, seed=9).copy()
    x[1, 333] = np.float16(np.inf)
    got = to_f32(pkg.ops.linear(pk, to_dev(x, gpu), None, path=1))
    assert not np.isfinite(got[1]).any()
    assert np.isfinite(got[0]).all()
    assert max_rel_err(got[0:1], x[0:1].astype(np.float32) @ w.astype(np.float32)) <= TOL


def test_activation_view_off_a_16_byte_boundary_is_copied(pkg, oracle, gpu):
    """x that starts 2 bytes into its storage (a contiguous view): the host side hands the kernels
    an aligned copy, the result is that of the aligned tensor bit for bit; the C entry point
    itself refuses such a pointer."""
    import ctypes
    K, N, M = 1024, 512, 3
    qw, qz, sc, _ = oracle.make_gptq(K, N, 128, seed=4, sym=False)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), None, 128, 0)
    flat = torch.randn(M * K + 1, dtype=torch.float16, device=gpu)
    x_off = flat[1:].view(M, K)
    assert x_off.is_contiguous() and x_off.data_ptr() % 16 != 0
    assert torch.equal(pkg.ops.linear(pk, x_off), pkg.ops.linear(pk, x_off.clone()))
    L = pkg._lib
    y = torch.empty((M, N), dtype=torch.float16, device=gpu)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=gpu)
    rc = L.load().q4_linear(ctypes.byref(pk.struct()), x_off.data_ptr(), None, y.data_ptr(), M, 0, ws.data_ptr(), ws.numel(), None)
    assert rc == L.ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("zeros_sym", [True, False])
def test_act_order_prefill_tall_tiles(pkg, oracle, gpu, dtype, zeros_sym):
    """288 tiles of 128 x 128 would be two rounds of the chip, 160 tiles of 256 x 128 are one: the act-order
    prefill kernel takes the 256-row tiles (last row tile ragged).  One-hot rows read the dequantized
    weights back bit for bit, random activations match the oracle."""
    K, N, M, gs = 512, 4096, 1100, 128
    bf = dtype == "bf16"
    qw, qz, sc, gi = oracle.make_gptq(K, N, gs, seed=21, sym=zeros_sym, act_order=True)
    w = oracle.dequant_gptq(qw, qz, sc, gi, gs, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), gs, 0)
    assert pkg.ops.select_path(pk, M, torch.bfloat16 if bf else torch.float16) == "gemm"
    ks = np.random.default_rng(5).integers(0, K, size=M)
    x = torch.zeros((M, K), dtype=torch.bfloat16 if bf else torch.float16, device=gpu)
    x[torch.arange(M, device=gpu), torch.as_tensor(ks, device=gpu)] = 1.0
    y = pkg.ops.linear(pk, x)
    torch.cuda.synchronize()
    got = y.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, w[ks].view(np.uint16))
    _run(pkg, oracle, gpu, K, N, gs, M, dtype=dtype, sym=zeros_sym, act=True, bias=True, seed=33)
