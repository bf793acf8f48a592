from .sparsegpt import SparseGPTModifier  # noqa: F401
