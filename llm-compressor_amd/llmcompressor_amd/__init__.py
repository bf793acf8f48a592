"""MI355X-native calibration-time quantization hot path (GPTQ, observers, packing).

``from llmcompressor_amd import oneshot`` mirrors ``from llmcompressor import oneshot``.
"""
__version__ = "0.1.0"


def __getattr__(name):
    if name == "oneshot":
        from .entrypoints import oneshot

        return oneshot
    if name == "active_session":
        from .core import active_session

        return active_session
    raise AttributeError(name)
