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
