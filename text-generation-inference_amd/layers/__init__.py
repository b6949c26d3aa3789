"""Host-side mirror of the reference's quantized-linear surface (layers/gptq, layers/awq)."""

from .linear import get_linear  # noqa: F401
