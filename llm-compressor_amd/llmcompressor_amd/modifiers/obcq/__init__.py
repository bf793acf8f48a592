"""``llmcompressor.modifiers.obcq``: the older home of ``SparseGPTModifier`` (reference: modifiers/obcq/__init__.py
re-exports ``sgpt_base``)."""
from ..pruning.sparsegpt import SparseGPTModifier  # noqa: F401

__all__ = ["SparseGPTModifier"]
