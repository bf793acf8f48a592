from . import gptq_quantize as _gptq_quantize
from .base import GPTQModifier  # noqa: F401
from .gptq_quantize import *  # noqa: F401,F403

__all__ = ["GPTQModifier"] + list(_gptq_quantize.__all__)
