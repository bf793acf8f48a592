from .base import SparseGPTModifier  # noqa: F401
