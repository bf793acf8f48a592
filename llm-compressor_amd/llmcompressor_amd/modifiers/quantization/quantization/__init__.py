from .base import QuantizationModifier  # noqa: F401
from .mixin import QuantizationMixin  # noqa: F401
