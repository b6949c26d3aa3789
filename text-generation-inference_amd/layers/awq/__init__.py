"""AWQ surface: WQLinear and the layout conversion helpers."""

from .quantize import WQLinear  # noqa: F401
