"""Old import location of the GPTQ modifier, kept with a deprecation warning
(reference: src/llmcompressor/modifiers/quantization/gptq/__init__.py)."""
import warnings as _warnings

from ...gptq import *  # noqa: F401,F403
from ...gptq import __all__ as _names

_warnings.warn(
    f"{__name__.rsplit('.modifiers', 1)[0]}.modifiers.quantization.gptq is a deprecated import location; "
    "import GPTQModifier from the modifiers.gptq package instead.",
    DeprecationWarning,
    stacklevel=2,
)
__all__ = list(_names)
