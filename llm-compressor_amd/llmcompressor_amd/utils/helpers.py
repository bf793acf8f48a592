"""``from llmcompressor.utils.helpers import calibration_forward_context, DisableQuantization`` (reference:
utils/helpers.py:120-170); the context managers are defined beside the pipelines that use them."""

__all__ = ["calibration_forward_context", "DisableQuantization"]


def __getattr__(name):
    if name in __all__:
        from .. import pipelines

        return getattr(pipelines, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
