"""Save-time integration with transformers models (reference: src/llmcompressor/transformers/)."""


def __getattr__(name):
    if name == "oneshot":  # the older import path: ``from llmcompressor.transformers import oneshot``
        from ..entrypoints import oneshot

        return oneshot
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
