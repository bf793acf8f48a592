from .quantization import QuantizationMixin, QuantizationModifier  # noqa: F401
from .calibration import *  # noqa: F401,F403


def __getattr__(name):
    # `from llmcompressor.modifiers.quantization import GPTQModifier` keeps working, as in the reference
    if name == "GPTQModifier":
        from ..gptq import GPTQModifier

        return GPTQModifier
    raise AttributeError(name)
