"""Golden fixtures (tests/golden/*.npz): the oracle must keep reproducing them, and on the
GPU the HIP kernels must reproduce them too (weights bit-exact, outputs within 2e-3)."""

from pathlib import Path

import numpy as np
import pytest
import torch

from tests.util import bits_of, max_rel_err, to_dev, to_f32

GOLDEN = sorted((Path(__file__).resolve().parent / "golden").glob("*.npz"))


def _load(path):
    d = np.load(path)
    K, N, gs, M, awq, bf = d["meta"].tolist()
    return d, K, N, gs, M, bool(awq), "bf16" if bf else "f16"


@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: p.stem)
def test_oracle_reproduces_golden(oracle, path):
    d, K, N, gs, M, awq, dtype = _load(path)
    gi = d["g_idx"] if "g_idx" in d else None
    if awq:
        w = oracle.dequant_awq(d["qweight"], d["qzeros"], d["scales"], gs, dtype)
    else:
        w = oracle.dequant_gptq(d["qweight"], d["qzeros"], d["scales"], gi, gs, dtype)
    wb = w.view(np.uint16) if w.dtype == np.float16 else w
    assert np.array_equal(wb, d["w_bits"])
    x = d["x"]
    y32, _ = oracle.linear_forward(x, w, None, dtype)
    assert np.array_equal(y32, d["y32"])


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=lambda p: p.stem)
def test_kernels_reproduce_golden(pkg, gpu, path):
    d, K, N, gs, M, awq, dtype = _load(path)
    bf = dtype == "bf16"
    gi = to_dev(d["g_idx"], gpu) if "g_idx" in d else None
    pk = pkg.ops.make_packed(to_dev(d["qweight"], gpu), to_dev(d["qzeros"], gpu), to_dev(d["scales"], gpu),
                             gi, gs, 1 if awq else 0)
    tdt = torch.bfloat16 if bf else torch.float16
    assert np.array_equal(bits_of(pkg.ops.dequantize(pk, tdt)), d["w_bits"])
    y = pkg.ops.linear(pk, to_dev(d["x"], gpu, bf16=bf), None)
    assert max_rel_err(to_f32(y), d["y32"]) <= (8e-3 if bf else 2e-3)
