"""``from llmcompressor.modeling.moe.linear_experts import LinearExperts2D`` (reference:
modeling/moe/linear_experts.py); the classes live in the package module."""
from . import ExpertMLP, LinearExperts2D, Llama4LinearExperts  # noqa: F401

__all__ = ["LinearExperts2D", "ExpertMLP", "Llama4LinearExperts"]
