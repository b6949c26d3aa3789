"""ctypes binding of libq4linear.so (declared in include/q4_linear.h).

The library is the only compute path of this package: if it is missing, loading fails
with an error that says how to build it; nothing falls back to PyTorch or the CPU.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_int, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "libq4linear.so"

LAYOUT_GPTQ = 0
LAYOUT_AWQ = 1
DTYPE_F16 = 0
DTYPE_BF16 = 1
DTYPE_F32 = 2  # gating logits of the mixture-of-experts router only
PATH_AUTO = 0
PATH_GEMV = 1
PATH_GEMM = 2
PATH_GENERIC = 3
PATH_NAMES = {PATH_GEMV: "gemv", PATH_GEMM: "gemm", PATH_GENERIC: "generic"}
WORKSPACE_COUNTER_BYTES = 4210688

ERR_INVALID_ARGUMENT = -1
ERR_UNSUPPORTED = -2
ERR_WORKSPACE = -3
ERR_LAUNCH = -4

# Q4_ACT_*: the MLP activations the fused gate_up epilogue knows, by the names the reference's
# configs use (hidden_act)
ACTIVATIONS = {"silu": 0, "gelu_fast": 1, "gelu_pytorch_tanh": 1, "gelu_tanh": 1, "gelu": 2}


class Q4Weight(Structure):
    """Mirror of `struct q4_weight`."""

    _fields_ = [
        ("qweight", c_void_p),
        ("qzeros", c_void_p),
        ("scales", c_void_p),
        ("g_idx", c_void_p),
        ("K", c_int32),
        ("N", c_int32),
        ("groupsize", c_int32),
        ("num_groups", c_int32),
        ("layout", c_int32),
    ]


class Q4MoeWeight(Structure):
    """Mirror of `struct q4_moe_weight`: expert 0's view plus the strides to the next expert."""

    _fields_ = [
        ("expert0", Q4Weight),
        ("num_experts", c_int32),
        ("qweight_stride", c_int64),
        ("qzeros_stride", c_int64),
        ("scales_stride", c_int64),
        ("g_idx_stride", c_int64),
    ]


# name -> (restype, argtypes); the single source for binding and for the export test
SIGNATURES = {
    "q4_abi_version": (c_int, []),
    "q4_last_error": (c_char_p, []),
    "q4_dequant": (c_int, [POINTER(Q4Weight), c_void_p, c_int, c_void_p]),
    "q4_linear": (
        c_int,
        [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "q4_linear_ex": (
        c_int,
        [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "q4_gemv_tuned": (
        c_int,
        [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "q4_gemv_candidates": (c_int, [POINTER(Q4Weight), c_int, c_int, POINTER(c_int32), c_int]),
    "q4_gemv_tuned_workspace_bytes": (c_size_t, [POINTER(Q4Weight), c_int, c_int, c_int, c_int, c_int, c_int]),
    "q4_linear_gate_up": (
        c_int,
        [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "q4_linear_gate_up_plan": (c_int, [POINTER(Q4Weight), c_int, c_int, POINTER(c_int)]),
    "q4_act_mul": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "q4_gptq_make_sequential": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "q4_gather_columns": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "q4_linear_perm": (c_int, [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                c_size_t, c_int, c_void_p]),
    "q4_workspace_bytes_perm": (c_size_t, [c_int, c_int, c_int]),
    "q4_linear_gate_up_perm": (c_int, [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                        c_void_p, c_size_t, c_void_p]),
    "q4_gptq_solve_block": (c_int, [c_void_p] * 7 + [c_int] * 7 + [c_void_p]),
    "q4_moe_gather_columns": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "q4_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "q4_select_path": (c_int, [POINTER(Q4Weight), c_int, c_int]),
    "q4_workspace_bytes_for": (c_size_t, [POINTER(Q4Weight), c_int]),
    "q4_linear_plan": (c_int, [POINTER(Q4Weight), c_int, c_int, POINTER(c_int), POINTER(c_size_t)]),
    "q4_noalloc_init": (c_int, []),
    "q4_linear_noalloc": (c_int, [POINTER(Q4Weight), c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "q4_moe_route": (
        c_int,
        [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "q4_moe_route_grouped": (
        c_int,
        [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "q4_moe_linear": (
        c_int,
        [POINTER(Q4MoeWeight), c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "q4_moe_linear_gate_up": (
        c_int,
        [POINTER(Q4MoeWeight), c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "q4_moe_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "q4_moe_workspace_bytes": (c_size_t, [POINTER(Q4MoeWeight), c_int, c_int]),
}

_lib = None


class Q4Error(RuntimeError):
    """A libq4linear call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libq4linear error {code}: {message}")
        self.code = code


def load() -> ctypes.CDLL:
    """Load (once) and return the bound library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python {HERE / 'build.py'}` "
            "(hipcc --offload-arch=gfx950); there is no fallback path"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int) -> None:
    if code < 0:
        raise Q4Error(code, load().q4_last_error().decode())
