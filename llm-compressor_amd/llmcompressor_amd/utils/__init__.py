"""``from llmcompressor.utils import load_context, dispatch_for_generation`` (reference: utils/__init__.py)."""

__all__ = ["load_context", "dispatch_for_generation", "get_main_device", "calibration_forward_context",
           "DisableQuantization"]


def __getattr__(name):
    if name in __all__:  # resolved on first use: utils is imported early, the pipelines late
        from . import dev, helpers

        return getattr(helpers if name in helpers.__all__ else dev, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
