"""The GPTQ solver (the reference's GPTQ.fasterquant, layers/gptq/quantize.py:243-351).

The oracle's float64 restatement is pinned by what the mathematics fixes, not by itself:
* with a diagonal Hessian no error is fed forward and every column is rounded to nearest with
  its group's range (closed form);
* whatever the rounding decisions, dW = W - Q satisfies dW H dW^T = sum of the squared fed-forward
  errors, row by row, H the damped (permuted) Hessian: the algebra behind the Cholesky form of the
  update (a transposed factor, a wrong divisor or a dropped update term breaks it);
* on correlated inputs the output error ||dW X|| is smaller than round-to-nearest's.
The GPU tests check the HIP kernel + host class against the same identity in fp32 and against
the oracle's decisions.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch


def calib(rng, K, n):
    """Correlated calibration inputs: a few strong shared directions plus noise."""
    basis = rng.standard_normal((8, K))
    X = rng.standard_normal((n, 8)) @ basis * 1.5 + 0.3 * rng.standard_normal((n, K))
    X[:, 5] *= 6.0
    return X


def rtn(oracle, W, gs, sym):
    K = W.shape[1]
    gs = K if gs == -1 else gs
    Q = np.zeros_like(W)
    for g in range(K // gs):
        blk = W[:, g * gs:(g + 1) * gs]
        s, z = oracle.gptq_find_params(blk, sym)
        Q[:, g * gs:(g + 1) * gs] = s[:, None] * (np.clip(np.rint(blk / s[:, None]) + z[:, None], 0, 15) - z[:, None])
    return Q


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("gs", [-1, 16])
def test_oracle_diagonal_hessian_is_round_to_nearest(oracle, gs, sym):
    rng = np.random.default_rng(3)
    W = rng.standard_normal((6, 64)) * 0.04
    H = np.diag(rng.uniform(0.5, 2.0, 64))
    Q, scale, zero, g_idx, err, _, _ = oracle.gptq_fasterquant(W, H, blocksize=16, groupsize=gs, sym=sym)
    assert np.array_equal(Q, rtn(oracle, W, gs, sym))
    assert np.array_equal(g_idx, np.arange(64) // (64 if gs == -1 else gs))


@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("gs,block", [(-1, 16), (16, 16), (8, 16), (32, 16)])
def test_oracle_error_identity_and_gain_over_round_to_nearest(oracle, gs, block, act_order):
    rng = np.random.default_rng(gs + block + act_order)
    rows, K, n = 7, 64, 300
    X = calib(rng, K, n)
    H = 2.0 / n * X.T @ X
    W = rng.standard_normal((rows, K)) * 0.05
    Q, scale, zero, g_idx, err, Hd, perm = oracle.gptq_fasterquant(
        W, H, blocksize=block, groupsize=gs, act_order=act_order, sym=False)
    d = (W - Q)[:, perm]
    lhs = np.einsum("ri,ij,rj->", d, Hd, d) / 2
    assert abs(lhs - err) <= 1e-10 * err
    # every value sits on its group's 16-level grid
    g = g_idx
    levels = np.rint(Q / scale[:, g] + zero[:, g])
    assert np.all((levels >= 0) & (levels <= 15))
    assert np.allclose(scale[:, g] * (levels - zero[:, g]), Q, rtol=0, atol=1e-12)
    if gs != -1 or not act_order:
        out_gptq = np.linalg.norm((W - Q) @ X.T)
        out_rtn = np.linalg.norm((W - rtn(oracle, W, gs, False)) @ X.T)
        assert out_gptq < out_rtn


def test_oracle_dead_inputs_and_act_order_permutation(oracle):
    rng = np.random.default_rng(9)
    rows, K, n = 4, 32, 100
    X = calib(rng, K, n)
    X[:, 11] = 0.0  # never active
    H = 2.0 / n * X.T @ X
    W = rng.standard_normal((rows, K)) * 0.05
    Q, _, _, g_idx, _, _, perm = oracle.gptq_fasterquant(W, H, blocksize=8, groupsize=8, act_order=True)
    assert np.all(Q[:, 11] == 0.0)
    assert np.all(np.diff(np.diag(np.where(np.eye(K) > 0, H, 0))[perm][:-1]) <= 1e-12)  # decreasing activity
    assert np.array_equal(np.sort(g_idx), np.arange(K) // 8)
    assert np.array_equal(g_idx[perm], np.arange(K) // 8)


def test_oracle_whole_row_range_includes_dead_input_columns(oracle):
    """groupsize -1: the row range is taken before dead columns are cleared (quantize.py:257-264),
    so an extreme weight in a dead input column still sets the row's scale."""
    rng = np.random.default_rng(4)
    rows, K, n = 3, 16, 50
    X = calib(rng, K, n)
    X[:, 5] = 0.0
    H = 2.0 / n * X.T @ X
    W = rng.standard_normal((rows, K)) * 0.05
    W[1, 5] = 3.0  # far outside the other weights of row 1
    _, scale, zero, _, _, _, _ = oracle.gptq_fasterquant(W, H, blocksize=8, groupsize=-1, sym=False)
    lo, hi = np.minimum(W.min(axis=1), 0), np.maximum(W.max(axis=1), 0)
    assert np.allclose(scale[:, 0], (hi - lo) / 15)
    assert scale[1, 0] > 0.19  # (3.0 - lo) / 15
    assert np.array_equal(zero[:, 0], np.rint(-lo / scale[:, 0]))


@pytest.mark.parametrize("sym", [True, False])
def test_oracle_mse_search_against_brute_force(oracle, sym):
    """The quantizer's grid search (quantize.py:101-123), restated here with plain loops over every
    candidate: first smallest sum of |q - x| ** 2.4 wins; sym keeps zero = 8; the unshrunk range
    is the first candidate, so the search never does worse than it."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((6, 40)) * 0.1
    x[2, 7] = 0.4    # an outlier
    x[4] = 0.0       # flat row
    scale, zero = oracle.gptq_find_params(x, sym, mse=True)
    s0, z0 = oracle.gptq_find_params(x, sym)
    for r in range(x.shape[0]):
        lo, hi = min(x[r].min(), 0.0), max(x[r].max(), 0.0)
        if sym:
            hi = max(abs(lo), hi)
            lo = -hi if lo < 0 else lo
        if lo == 0 and hi == 0:
            lo, hi = -1.0, 1.0
        best, pick = np.inf, None
        for i in range(80):
            p = 1 - i / 100
            sc = (p * hi - p * lo) / 15.0
            ze = 8.0 if sym else float(np.rint(-(p * lo) / sc))
            err = 0.0
            for v in x[r]:
                q = sc * (min(max(float(np.rint(v / sc)) + ze, 0.0), 15.0) - ze)
                err += abs(q - v) ** 2.4
            if err < best:
                best, pick = err, (sc, ze)
        assert np.isclose(scale[r], pick[0], rtol=1e-12) and zero[r] == pick[1]
        plain = np.sum(np.abs(oracle._gptq_round(x[r], s0[r], z0[r]) - x[r]) ** 2.4)
        assert best <= plain + 1e-15
    assert np.all(scale <= s0 * (1 + 1e-12)) and np.sum(scale < s0) >= 2  # ranges only shrink, and some do
    assert scale[4] == s0[4]  # a flat row keeps its unit range (every candidate has zero error)


# --------------------------------------------------------------------------- GPU


def _solve(pkg, gpu, W, X, gs, act_order, sym, block=128):
    lin = torch.nn.Linear(W.shape[1], W.shape[0], bias=False)
    lin.weight.data = torch.from_numpy(W.astype(np.float32))
    lin = lin.to(gpu)
    solver = pkg.GPTQ(lin, sym=sym)
    xt = torch.from_numpy(X.astype(np.float32)).to(gpu)
    half = X.shape[0] // 2
    solver.add_batch(xt[:half].unsqueeze(0), None)   # two batches: the running mean is exercised
    solver.add_batch(xt[half:].unsqueeze(0), None)
    H = solver.H.double().cpu().numpy()
    scale, zero, g_idx, err = solver.fasterquant(blocksize=block, groupsize=gs, act_order=act_order)
    return lin.weight.data.double().cpu().numpy(), scale.double().cpu().numpy(), zero.double().cpu().numpy(), \
        g_idx.cpu().numpy(), err, H


@pytest.mark.gpu
@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("rows,K,gs,block", [(37, 256, 128, 128), (64, 384, 64, 128), (16, 256, -1, 128),
                                             (33, 512, 256, 128), (20, 200, 40, 100), (8, 128, 32, 128)])
def test_gpu_solver_identity_and_oracle_agreement(pkg, oracle, gpu, rows, K, gs, block, act_order, sym):
    rng = np.random.default_rng(rows + K + act_order)
    n = 2 * K
    X = calib(rng, K, n)
    W = rng.standard_normal((rows, K)) * 0.05
    Q, scale, zero, g_idx, err, H = _solve(pkg, gpu, W, X, gs, act_order, sym, block)
    # the Hessian the class accumulated (two batches, each counted as one sample like the
    # reference's 3-D batches) is proportional to X^T X
    ref_H = X.T @ X
    assert np.allclose(H / H[0, 0], ref_H / ref_H[0, 0], rtol=2e-4, atol=2e-4)
    oQ, oscale, ozero, og_idx, oerr, Hd, perm = oracle.gptq_fasterquant(
        W.astype(np.float32), H, blocksize=block, groupsize=gs, act_order=act_order, sym=sym)
    assert np.array_equal(g_idx, og_idx)
    # identity in fp32: dW H dW^T / 2 = error
    d = (W.astype(np.float32).astype(np.float64) - Q)[:, perm]
    lhs = np.einsum("ri,ij,rj->", d, Hd, d) / 2
    assert abs(lhs - err) <= 2e-3 * err
    # same decisions as the float64 oracle except near rounding ties, same error
    g = g_idx
    lv = np.rint(Q / scale[:, g] + zero[:, g])
    olv = np.rint(oQ / oscale[:, g] + ozero[:, g])
    assert np.mean(lv == olv) >= 0.97
    assert abs(err - oerr) <= 2e-2 * oerr
    assert np.allclose(scale, oscale, rtol=2e-2, atol=1e-7) and np.mean(zero == ozero) >= 0.97


@pytest.mark.gpu
@pytest.mark.parametrize("sym", [True, False])
def test_gpu_solver_whole_row_range_with_dead_input(pkg, oracle, gpu, sym):
    """groupsize -1 with an all-zero calibration column that holds a row's extreme weight."""
    rng = np.random.default_rng(12)
    rows, K, n = 8, 128, 64
    X = calib(rng, K, n)
    X[:, 17] = 0.0
    W = rng.standard_normal((rows, K)) * 0.05
    W[2, 17] = 2.5
    Q, scale, zero, _, _, H = _solve(pkg, gpu, W, X, -1, False, sym)
    _, s_ref, z_ref, _, _, _, _ = oracle.gptq_fasterquant(W.astype(np.float32).astype(np.float64), H, groupsize=-1, sym=sym)
    assert np.allclose(scale[:, 0], s_ref[:, 0], rtol=1e-6)
    assert np.array_equal(zero[:, 0], z_ref[:, 0])
    assert np.all(Q[:, 17] == 0.0)


@pytest.mark.gpu
@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("gs", [64, 256, -1])
def test_gpu_solver_mse_ranges(pkg, oracle, gpu, gs, sym):
    """mse=True: the ranges found on the GPU (fp32) against the oracle's search (float64) on the
    same weights, then a whole solve against the oracle's.  Near-ties between neighbouring shrink factors may fall the other way in
    fp32: nearly all (row, group) pairs agree exactly, the rest by one grid step."""
    rng = np.random.default_rng(31)
    rows, K, n = 24, 256, 96
    X = calib(rng, K, n)
    W = rng.standard_normal((rows, K)) * 0.05
    W[rng.integers(0, rows, 12), rng.integers(0, K, 12)] *= 8.0  # outliers
    w32 = W.astype(np.float32).astype(np.float64)
    t = torch.from_numpy(w32.astype(np.float32)).to(gpu)
    s_gpu, z_gpu = pkg.layers.gptq.solver.find_params(t, sym, True)
    s_ref, z_ref = oracle.gptq_find_params(w32, sym, mse=True)
    close = np.isclose(s_gpu.double().cpu().numpy(), s_ref, rtol=1e-5)
    assert close.mean() >= 0.9
    assert np.all(np.abs(s_gpu.double().cpu().numpy() / s_ref - 1) <= 0.012)  # at most a grid step apart
    # the whole solve with the searched ranges satisfies the solver's identity and beats min/max
    lin = torch.nn.Linear(K, rows, bias=False)
    lin.weight.data = torch.from_numpy(w32.astype(np.float32))
    lin = lin.to(gpu)
    solver = pkg.GPTQ(lin, sym=sym, mse=True)
    solver.add_batch(torch.from_numpy(X.astype(np.float32)).to(gpu).unsqueeze(0), None)
    H = solver.H.double().cpu().numpy()
    scale, zero, g_idx, err = solver.fasterquant(groupsize=gs)
    Q = lin.weight.data.double().cpu().numpy()
    G = scale.shape[1]
    sc, ze = scale.double().cpu().numpy(), zero.double().cpu().numpy()
    g = g_idx.cpu().numpy()
    levels = np.rint(Q / sc[:, g] + ze[:, g])
    assert np.all((levels >= 0) & (levels <= 15))
    assert np.allclose(sc[:, g] * (levels - ze[:, g]), Q, atol=1e-6)
    # (the search minimises an unweighted |.|^2.4 norm, so the Hessian-weighted error need not
    # drop against min/max ranges; it must match the oracle's solve with the same search)
    _, s_or, z_or, _, err_or, _, _ = oracle.gptq_fasterquant(w32, H, groupsize=gs, sym=sym, mse=True)
    assert abs(err - err_or) <= 0.1 * err_or
    assert np.isclose(sc, s_or, rtol=1e-4).mean() >= 0.8


@pytest.mark.gpu
def test_gpu_solver_output_packs_and_runs(pkg, oracle, gpu):
    """Solver -> QuantLinear.pack -> kernels: the layer reproduces the solver's weights and beats
    round-to-nearest on the calibration inputs."""
    rng = np.random.default_rng(21)
    rows, K, gs = 128, 512, 128
    X = calib(rng, K, 1024)
    W = rng.standard_normal((rows, K)) * 0.05
    for act_order in (False, True):
        Q, scale, zero, g_idx, err, H = _solve(pkg, gpu, W, X, gs, act_order, False)
        layer = pkg.QuantLinear.new(4, gs, K, rows, bias=False)
        from types import SimpleNamespace
        layer.pack(SimpleNamespace(weight=torch.from_numpy(Q.astype(np.float32)), bias=None),
                   torch.from_numpy(scale.astype(np.float32)), torch.from_numpy(zero.astype(np.float32)),
                   torch.from_numpy(g_idx))
        layer = layer.to(gpu)
        dense = layer.dequantize().float().cpu().numpy()  # [K, rows]
        assert np.allclose(dense.T, Q, rtol=2e-3, atol=1e-5)  # fp16 scales
        x = torch.from_numpy(X[:64].astype(np.float16)).to(gpu)
        y = layer(x).float().cpu().numpy()
        want = X[:64].astype(np.float16).astype(np.float64) @ W.T
        out_rtn = np.linalg.norm(X[:64] @ (W - rtn(oracle, W, gs, False)).T)
        assert np.linalg.norm(y - want) < out_rtn


@pytest.mark.gpu
def test_gpu_solver_rejects_cpu_layers_and_bad_blocks(pkg, gpu):
    lin = torch.nn.Linear(64, 8, bias=False)
    s = pkg.GPTQ(lin)
    s.add_batch(torch.randn(1, 4, 64))
    with pytest.raises(RuntimeError, match="GPU only"):
        s.fasterquant()
    lib = pkg._lib.load()
    t = torch.zeros(64 * 64, device=gpu)
    assert lib.q4_gptq_solve_block(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(),
                                   t.data_ptr(), 8, 64, 0, 129, -1, 1, 1, None) == pkg._lib.ERR_INVALID_ARGUMENT


@pytest.mark.gpu
@pytest.mark.parametrize("act_order,gs,sym", [(False, 128, False), (True, 128, False), (False, -1, True), (True, 64, True)])
def test_quantize_linear_end_to_end(pkg, oracle, gpu, act_order, gs, sym):
    """Calibrate -> solve -> pack -> run: the quantized layer tracks the dense one on held-out
    inputs of the calibration distribution better than round-to-nearest does."""
    rng = np.random.default_rng(4)
    rows, K = 192, 512
    X = calib(rng, K, 2048)
    W = rng.standard_normal((rows, K)) * 0.05
    lin = torch.nn.Linear(K, rows, bias=True)
    lin.weight.data = torch.from_numpy(W.astype(np.float32))
    b = lin.bias.data.clone()
    lin = lin.to(gpu)
    layer, err = pkg.quantize_linear(lin, torch.from_numpy(X[:1536].astype(np.float32)).to(gpu), groupsize=gs,
                                     act_order=act_order, sym=sym)
    assert type(layer).__name__ == "QuantLinear" and err > 0
    held = X[1536:1600]
    y = layer(torch.from_numpy(held.astype(np.float16)).to(gpu)).float().cpu().numpy()
    want = held.astype(np.float16).astype(np.float64) @ W.T + b.numpy()
    out_rtn = np.linalg.norm(held @ (W - rtn(oracle, W, gs, sym)).T)
    assert np.linalg.norm(y - want) < out_rtn
