"""``from llmcompressor.modeling.moe.context import moe_calibration_context`` (reference:
modeling/moe/context.py)."""
from . import get_calibrate_all_experts_flag, moe_calibration_context  # noqa: F401

__all__ = ["moe_calibration_context", "get_calibrate_all_experts_flag"]
