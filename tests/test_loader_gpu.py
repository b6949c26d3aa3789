"""End to end on the GPU: safetensors checkpoint -> loader -> get_linear -> forward.

Every shard's output is compared with the oracle on that shard's slice of the dense
matrix; row shards are additionally summed (what the all-reduce after a row-parallel
layer would produce) and compared with the unsharded product.
"""

from types import SimpleNamespace

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from tests.util import max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu

TOL = 2e-3
K, N, GS = 2048, 1536, 128


def group(rank, size):
    return SimpleNamespace(rank=lambda: rank, size=lambda: size)


def i32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32).copy())


def checkpoint(oracle, tmp_path, layout, act_order=False, seed=21):
    if layout == "awq":
        qw, qz, sc = oracle.make_awq(K, N, GS, seed=seed)
        dense = oracle.dequant_awq(qw, qz, sc, GS)
        t = {"proj.qweight": i32(qw), "proj.qzeros": i32(qz), "proj.scales": torch.from_numpy(sc)}
    else:
        qw, qz, sc, gi = oracle.make_gptq(K, N, GS, seed=seed, sym=False, act_order=act_order)
        dense = oracle.dequant_gptq(qw, qz, sc, gi, GS)
        stored = gi if gi is not None else (np.arange(K) // GS).astype(np.int32)
        t = {"proj.qweight": i32(qw), "proj.qzeros": i32(qz), "proj.scales": torch.from_numpy(sc),
             "proj.g_idx": torch.from_numpy(stored)}
    path = tmp_path / "model.safetensors"
    save_file(t, str(path))
    return path, dense


def loader_for(pkg, quantize, quant_method, desc_act=False):
    return pkg.GPTQWeightsLoader(bits=4, groupsize=GS, desc_act=desc_act, quant_method=quant_method,
                                 quantize=quantize, sym=False, modules_to_not_convert=[])


CASES = [
    ("gptq", "gptq", "gptq", False),
    ("gptq", "gptq", "gptq", True),
    ("awq", "awq", "awq", False),
    ("awq", "gptq", "awq", False),   # AWQ file repacked to the GPTQ layout at load time
]


@pytest.mark.parametrize("layout,quantize,quant_method,act", CASES)
@pytest.mark.parametrize("M", [1, 48])
def test_column_and_row_shards_forward(pkg, oracle, gpu, tmp_path, layout, quantize, quant_method, act, M):
    path, dense = checkpoint(oracle, tmp_path, layout, act)
    loader = loader_for(pkg, quantize, quant_method, desc_act=act)
    x = oracle.make_x(M, K, seed=5)
    y_full, _ = oracle.linear_forward(x, dense, None, "f16")
    xt = to_dev(x, gpu)
    world = 2
    row_sum = np.zeros((M, N), dtype=np.float32)
    for rank in range(world):
        weights = pkg.Weights([path], gpu, torch.float16, group(rank, world), loader)
        col = pkg.get_linear(weights.get_weights_col("proj"), None)
        got = to_f32(col(xt))
        want = y_full[:, rank * N // world:(rank + 1) * N // world]
        assert max_rel_err(got, want) <= TOL

        row = pkg.get_linear(weights.get_weights_row("proj"), None)
        ks = slice(rank * K // world, (rank + 1) * K // world)
        got = to_f32(row(xt[:, ks].contiguous()))
        want, _ = oracle.linear_forward(x[:, ks], dense[ks], None, "f16")
        assert max_rel_err(got, want) <= TOL
        row_sum += got
    torch.cuda.synchronize()
    assert max_rel_err(row_sum, y_full) <= TOL

    whole = pkg.get_linear(pkg.Weights([path], gpu, torch.float16, None, loader).get_weights("proj"), None)
    assert max_rel_err(to_f32(whole(xt)), y_full) <= TOL


def test_packed_gate_up_forward(pkg, oracle, gpu, tmp_path):
    path, dense = checkpoint(oracle, tmp_path, "gptq")
    loader = loader_for(pkg, "gptq", "gptq")
    x = oracle.make_x(4, K, seed=6)
    y_full, _ = oracle.linear_forward(x, dense, None, "f16")
    for rank in range(2):
        weights = pkg.Weights([path], gpu, torch.float16, group(rank, 2), loader)
        layer = pkg.get_linear(weights.get_weights_col_packed_gate_up("proj"), None)
        got = to_f32(layer(to_dev(x, gpu)))
        q = N // 4
        want = np.concatenate([y_full[:, rank * q:(rank + 1) * q],
                               y_full[:, 2 * q + rank * q: 2 * q + (rank + 1) * q]], axis=1)
        assert max_rel_err(got, want) <= TOL


@pytest.mark.parametrize("act_order", [True, False])
def test_solver_made_checkpoint_through_the_loader(pkg, oracle, gpu, tmp_path, act_order):
    """The route a self-quantized model takes: GPTQ solve and pack one layer with act-order
    (`quantize_linear`), write its tensors the way the reference's quantizer saves them
    (server/text_generation_server/layers/gptq/quantize.py:957-1012: the module's state dict plus
    the `gptq_bits` / `gptq_groupsize` / `gptq_sym` marker tensors, and a quantize config beside
    it), read the directory back with `get_loader("gptq")` -> `Weights` -> `get_linear`, and run
    it.  The g_idx here is the solver's (groups in order of the Hessian diagonal), not a random
    permutation.  Bars: the loaded layer reproduces the in-memory packed layer bit for bit, and
    it tracks the dense layer on held-out inputs better than round-to-nearest does."""
    import json

    rng = np.random.default_rng(12)
    K2, N2, gs = 1024, 384, 128
    # correlated calibration inputs (a few strong shared directions plus noise: what the solver's
    # error feedback exploits) with very different column scales, so that act-order reorders
    basis = rng.standard_normal((8, K2))
    col_scale = np.exp(rng.standard_normal(K2))
    X = ((rng.standard_normal((2048, 8)) @ basis * 1.5 + 0.3 * rng.standard_normal((2048, K2))) * col_scale).astype(np.float32)
    W = (rng.standard_normal((N2, K2)) * 0.05).astype(np.float32)
    lin = torch.nn.Linear(K2, N2, bias=True)
    lin.weight.data = torch.from_numpy(W.copy())
    bias = lin.bias.data.clone()
    lin = lin.to(gpu)
    layer, err = pkg.quantize_linear(lin, torch.from_numpy(X[:1536]).to(gpu), groupsize=gs, act_order=act_order, sym=True)
    g_idx = layer.g_idx.cpu()
    trivial = bool(torch.equal(g_idx, (torch.arange(K2) // gs).to(g_idx.dtype)))
    assert trivial != act_order, "act-order must reorder the rows of this calibration set (and only act-order)"

    model_dir = tmp_path / "quantized"
    model_dir.mkdir()
    tensors = {f"model.proj.{k}": v.detach().cpu().contiguous() for k, v in layer.state_dict().items()}
    tensors.update({"gptq_bits": torch.tensor(4), "gptq_groupsize": torch.tensor(gs), "gptq_sym": torch.tensor(True)})
    save_file(tensors, str(model_dir / "model.safetensors"))
    (model_dir / "quantize_config.json").write_text(json.dumps(
        {"bits": 4, "group_size": gs, "desc_act": act_order, "sym": True, "quant_method": "gptq"}))

    loader = pkg.get_loader("gptq", str(model_dir))
    weights = pkg.Weights([model_dir / "model.safetensors"], gpu, torch.float16, None, loader)
    loaded = pkg.get_linear(weights.get_weights("model.proj"), weights.get_tensor("model.proj.bias"))

    held = X[1536:1600]
    xt = torch.from_numpy(held.astype(np.float16)).to(gpu)
    for M in (1, 16, 64):
        assert torch.equal(loaded(xt[:M]), layer(xt[:M])), f"loaded layer differs from the packed one at M={M}"
    y = to_f32(loaded(xt))
    want = held.astype(np.float16).astype(np.float64) @ W.T.astype(np.float64) + bias.numpy()
    # round-to-nearest with the same grid, for the bar
    Wg = W.reshape(N2, K2 // gs, gs)
    absmax = np.abs(Wg).max(axis=2, keepdims=True)
    scale = np.maximum(absmax, 1e-9) * 2 / 15
    rtn = (np.clip(np.round(Wg / scale) + 8, 0, 15) - 8) * scale
    out_rtn = np.linalg.norm(held.astype(np.float64) @ (W - rtn.reshape(N2, K2)).T)
    assert np.linalg.norm(y - want) < out_rtn
