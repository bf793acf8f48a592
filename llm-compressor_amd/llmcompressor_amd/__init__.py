"""MI355X-native calibration-time quantization hot path (GPTQ, observers, packing).

``from llmcompressor_amd import oneshot, model_free_ptq`` mirrors ``from llmcompressor import oneshot, model_free_ptq``.
"""
__version__ = "0.1.0"


def __getattr__(name):
    if name == "oneshot":
        from .entrypoints import oneshot

        return oneshot
    if name == "model_free_ptq":
        from .entrypoints import model_free_ptq

        return model_free_ptq
    if name == "active_session":
        from .core import active_session

        return active_session
    raise AttributeError(name)
