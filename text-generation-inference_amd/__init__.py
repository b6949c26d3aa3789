"""MI355X-native int4 weight-only quantized linear layer (GPTQ / AWQ checkpoints).

Drop-in for the reference's `layers/gptq` and `layers/awq` surface: the same weight
container and module classes, backed by hand-written gfx950 HIP kernels reached through
the C ABI in include/q4_linear.h.  The directory name is not a Python identifier; load it
with `importlib.import_module("text-generation-inference_amd")` with the repository root
on sys.path.
"""

from . import _lib, ops  # noqa: F401
from .layers.linear import get_linear  # noqa: F401
from .layers.mlp import fold_down_permutation, gate_up_act  # noqa: F401
from .layers.gptq import (  # noqa: F401
    GPTQWeight,
    GPTQWeightsLoader,
    QuantLinear,
    ExllamaQuantLinear,
    create_exllama_buffers,
    set_device,
)
from .layers.awq.quantize import WQLinear  # noqa: F401
from .layers.gptq.solver import GPTQ, quantize_linear  # noqa: F401
from .layers.moe import GPTQSparseMoELayer, GPTQMoEWeight  # noqa: F401
from .layers.awq import conversion_utils  # noqa: F401
from .utils.weights import Weights, WeightsLoader, DefaultWeightsLoader, UnquantizedWeight  # noqa: F401
from .utils.quantization import get_loader, get_quantizer_config  # noqa: F401

__all__ = [
    "GPTQ",
    "GPTQWeight",
    "GPTQWeightsLoader",
    "Weights",
    "get_loader",
    "get_quantizer_config",
    "QuantLinear",
    "ExllamaQuantLinear",
    "WQLinear",
    "GPTQSparseMoELayer",
    "GPTQMoEWeight",
    "get_linear",
    "gate_up_act",
    "create_exllama_buffers",
    "set_device",
    "conversion_utils",
    "ops",
]
