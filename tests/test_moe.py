"""Oracle of the mixture-of-experts routing and block, pinned without a GPU."""

from __future__ import annotations

import numpy as np
import pytest
from scipy.special import softmax


def test_fused_topk_against_scipy_brute_force(oracle):
    rng = np.random.default_rng(0)
    for T, E, k in [(1, 8, 2), (7, 8, 1), (33, 64, 6), (5, 3, 3)]:
        g = rng.standard_normal((T, E)).astype(np.float32) * 3
        for renorm in (False, True):
            w, ids = oracle.moe_fused_topk(g, k, renorm)
            p = softmax(g.astype(np.float64), axis=1)
            for t in range(T):
                order = sorted(range(E), key=lambda e: (-p[t, e], e))[:k]
                assert ids[t].tolist() == order
                want = p[t, order] / (p[t, order].sum() if renorm else 1.0)
                assert np.allclose(w[t], want, rtol=2e-6, atol=1e-9)
            if renorm:
                assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)


def test_fused_topk_hand_case_and_ties(oracle):
    # two experts, logits ln(3) and 0: probabilities 3/4 and 1/4
    w, ids = oracle.moe_fused_topk(np.array([[np.log(3.0), 0.0]], dtype=np.float32), 2, False)
    assert ids.tolist() == [[0, 1]] and np.allclose(w, [[0.75, 0.25]], atol=1e-7)
    w, ids = oracle.moe_fused_topk(np.array([[np.log(3.0), 0.0]], dtype=np.float32), 1, True)
    assert ids.tolist() == [[0]] and np.allclose(w, [[1.0]])
    # equal logits: the lowest expert wins
    w, ids = oracle.moe_fused_topk(np.zeros((1, 4), dtype=np.float32), 2, True)
    assert ids.tolist() == [[0, 1]] and np.allclose(w, [[0.5, 0.5]])


def test_grouped_topk_brute_force_and_special_cases(oracle):
    rng = np.random.default_rng(4)
    for T, E, groups, keep, k in [(9, 16, 4, 2, 3), (5, 160, 8, 3, 6), (3, 8, 8, 4, 2), (4, 12, 3, 1, 4)]:
        g = (rng.standard_normal((T, E)) * 2).astype(np.float32)
        for renorm in (False, True):
            w, ids = oracle.moe_grouped_topk(g, k, renorm, groups, keep)
            p = softmax(g.astype(np.float64), axis=1)
            per = E // groups
            for t in range(T):
                gmax = [p[t, a * per:(a + 1) * per].max() for a in range(groups)]
                kept = sorted(range(groups), key=lambda a: (-gmax[a], a))[:keep]
                cand = [e for e in range(E) if e // per in kept]
                order = sorted(cand, key=lambda e: (-p[t, e], e))[:k]
                assert ids[t].tolist() == order
                want = p[t, order] / (p[t, order].sum() if renorm else 1.0)
                assert np.allclose(w[t], want, rtol=2e-6, atol=1e-9)
    # one group, or every group kept: plain top-k
    g = rng.standard_normal((6, 12)).astype(np.float32)
    for groups, keep in ((1, 1), (4, 4)):
        w, ids = oracle.moe_grouped_topk(g, 3, True, groups, keep)
        w0, ids0 = oracle.moe_fused_topk(g, 3, True)
        assert np.array_equal(ids, ids0) and np.allclose(w, w0)


def test_moe_forward_equals_the_dense_sum_over_all_experts(oracle):
    """Applying every expert to every token with zero weight for the ones not chosen (the
    reference's dense formulation) gives the same block output."""
    rng = np.random.default_rng(1)
    T, H, I, E, k = 5, 128, 256, 4, 2
    x = (rng.standard_normal((T, H)) * 0.5).astype(np.float16)
    gating = rng.standard_normal((T, E)).astype(np.float32)
    gu, dn = [], []
    for e in range(E):
        qw, qz, sc, _ = oracle.make_gptq(H, 2 * I, 64, seed=10 + e, sym=False)
        gu.append(oracle.dequant_gptq(qw, qz, sc, None, 64, "f16"))
        qw, qz, sc, _ = oracle.make_gptq(I, H, 64, seed=20 + e, sym=False)
        dn.append(oracle.dequant_gptq(qw, qz, sc, None, 64, "f16"))
    out32, out16 = oracle.moe_forward(x, gating, gu, dn, k, True, "silu", "f16")
    w, ids = oracle.moe_fused_topk(gating, k, True)
    dense = np.zeros((T, H), dtype=np.float32)
    for e in range(E):
        weight_e = np.zeros(T, dtype=np.float32)
        for t in range(T):
            for j in range(k):
                if ids[t, j] == e:
                    weight_e[t] = w[t, j]
        _, h = oracle.gate_up_forward(x, gu[e], "silu", None, "f16")
        _, d = oracle.linear_forward(h, dn[e], None, "f16")
        dense += weight_e[:, None] * d.astype(np.float32)
    assert np.allclose(out32, dense, rtol=1e-6, atol=1e-6)
    assert out16.dtype == np.float16 and out16.shape == (T, H)
