"""q4_linear_noalloc (the entry point that allocates nothing: its split-K scratch is a device
array built into the library) against q4_linear with a caller-provided workspace.

Both run the same kernels with the same decomposition, and every combine is order-independent
or in fixed order, so the outputs must agree bit for bit.  Two calls in a row share the
built-in array; the second is smaller, so it would see anything the first left behind."""

import ctypes

import numpy as np
import pytest
import torch

from tests.util import bits_of, max_rel_err, to_dev, to_f32

pytestmark = pytest.mark.gpu


def _both(pkg, oracle, gpu, K, N, M, layout="gptq", dtype="f16", act=False, seed=0):
    bf = dtype == "bf16"
    if layout == "gptq":
        qw, qz, sc, gi = oracle.make_gptq(K, N, 128, seed=seed, sym=False, act_order=act)
        w = oracle.dequant_gptq(qw, qz, sc, gi, 128, dtype)
        lay = 0
    else:
        qw, qz, sc = oracle.make_awq(K, N, 128, seed=seed)
        gi = None
        w = oracle.dequant_awq(qw, qz, sc, 128, dtype)
        lay = 1
    x = oracle.make_x(M, K, seed=seed + 1, dtype=dtype)
    y32, _ = oracle.linear_forward(x, w, None, dtype)
    pk = pkg.ops.make_packed(to_dev(qw, gpu), to_dev(qz, gpu), to_dev(sc, gpu), to_dev(gi, gpu), 128, lay)
    xt = to_dev(x, gpu, bf16=bf)
    want = pkg.ops.linear(pk, xt, None)  # q4_linear_ex with a torch workspace
    got = torch.full_like(want, float("nan"))
    lib = pkg._lib.load()
    st = pk.struct()
    before = torch.cuda.memory_allocated(gpu)
    rc = lib.q4_linear_noalloc(ctypes.byref(st), xt.data_ptr(), None, got.data_ptr(), M,
                               pkg._lib.DTYPE_BF16 if bf else pkg._lib.DTYPE_F16,
                               torch.cuda.current_stream(gpu).cuda_stream)
    pkg._lib.check(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(gpu) == before
    assert np.array_equal(bits_of(got), bits_of(want)), (K, N, M, layout, dtype)
    err = max_rel_err(to_f32(got), y32)
    assert err <= (8e-3 if bf else 2e-3), err


def test_noalloc_matches_q4_linear_two_calls_in_a_row(pkg, oracle, gpu):
    assert pkg._lib.load().q4_noalloc_init() == 0
    # decode with K split over workgroups (fixed-point cells), then a smaller decode problem
    _both(pkg, oracle, gpu, 4096, 4096, 1, seed=1)
    _both(pkg, oracle, gpu, 2048, 1024, 1, seed=2)
    # ticket path (several rows), then fewer rows on a smaller matrix
    _both(pkg, oracle, gpu, 14336, 4096, 8, seed=3)
    _both(pkg, oracle, gpu, 4096, 1024, 5, seed=4)
    # prefill: split-K partial tiles in the array, then a smaller prefill and a decode call
    _both(pkg, oracle, gpu, 4096, 1024, 256, seed=5)
    _both(pkg, oracle, gpu, 2048, 512, 96, seed=6)
    _both(pkg, oracle, gpu, 2048, 512, 1, seed=7)


@pytest.mark.parametrize("layout,act,dtype", [("awq", False, "f16"), ("gptq", True, "f16"), ("gptq", False, "bf16")])
def test_noalloc_other_layouts(pkg, oracle, gpu, layout, act, dtype):
    _both(pkg, oracle, gpu, 4096, 2048, 4, layout=layout, dtype=dtype, act=act, seed=11)
    _both(pkg, oracle, gpu, 1024, 512, 2, layout=layout, dtype=dtype, act=act, seed=12)


def test_noalloc_rejects_what_does_not_fit(pkg, gpu):
    """A decode problem whose partial sums exceed the built-in array is refused with a clear
    error before anything is launched (fake pointers: nothing dereferences them)."""
    L = pkg._lib
    lib = L.load()
    K, N = 32768, 65536
    w = L.Q4Weight(0x1000, 0x2000, 0x3000, None, K, N, 128, K // 128, 0)
    path, need = ctypes.c_int(0), ctypes.c_size_t(0)
    for m in range(1, 65):
        assert lib.q4_linear_plan(ctypes.byref(w), m, 0, ctypes.byref(path), ctypes.byref(need)) == 0
        if path.value == L.PATH_GEMV and need.value > 16777216:
            rc = lib.q4_linear_noalloc(ctypes.byref(w), 0x10, None, 0x20, m, 0, None)
            assert rc == L.ERR_WORKSPACE
            assert b"scratch" in lib.q4_last_error()
            return
    raise AssertionError("no decode problem of this shape exceeds the array: pick another shape")
