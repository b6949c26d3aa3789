"""Writes the small golden fixtures under tests/golden/ from the CPU oracle.

Run from the repository root: `python tests/golden/make_golden.py`.  The vectors are
produced by oracle/q4_oracle.py (itself pinned by tests/test_oracle.py); no reference
code is imported or run.  Each .npz holds the packed inputs, the activations, the
dequantized weight bit patterns and the fp32-accumulated output.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import q4_oracle as o  # noqa: E402

HERE = Path(__file__).resolve().parent

CASES = {
    # name: (layout, K, N, groupsize, sym, act_order, M, dtype)
    "gptq_sym_g128": ("gptq", 256, 64, 128, True, False, 3, "f16"),
    "gptq_asym_actorder_g32": ("gptq", 256, 64, 32, False, True, 5, "f16"),
    "gptq_asym_g64_bf16": ("gptq", 128, 64, 64, False, False, 2, "bf16"),
    "awq_g128": ("awq", 256, 64, 128, False, False, 4, "f16"),
}


def build(name):
    layout, K, N, gs, sym, act, M, dtype = CASES[name]
    seed = sum(map(ord, name))
    if layout == "gptq":
        qw, qz, sc, gi = o.make_gptq(K, N, gs, seed=seed, sym=sym, act_order=act)
        w = o.dequant_gptq(qw, qz, sc, gi, gs, dtype)
    else:
        qw, qz, sc = o.make_awq(K, N, gs, seed=seed)
        gi = None
        w = o.dequant_awq(qw, qz, sc, gs, dtype)
    x = o.make_x(M, K, seed=seed, dtype=dtype)
    y32, ycast = o.linear_forward(x, w, None, dtype)
    out = dict(
        qweight=qw, qzeros=qz, scales=sc, x=x,
        w_bits=w.view(np.uint16) if w.dtype == np.float16 else w,
        y32=y32, y_bits=ycast.view(np.uint16) if ycast.dtype == np.float16 else ycast,
        meta=np.array([K, N, gs, M, int(layout == "awq"), int(dtype == "bf16")], dtype=np.int64),
    )
    if gi is not None:
        out["g_idx"] = gi
    return out


if __name__ == "__main__":
    for name in CASES:
        np.savez_compressed(HERE / f"{name}.npz", **build(name))
        print("wrote", name)
