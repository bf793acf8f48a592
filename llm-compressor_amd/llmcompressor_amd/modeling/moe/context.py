"""``from llmcompressor.modeling.moe.context import moe_calibration_context`` (reference:
modeling/moe/context.py)."""
from . import moe_calibration_context  # noqa: F401

__all__ = ["moe_calibration_context"]
