"""``from llmcompressor.modeling.moe.linearize import linearize_moe`` (reference: modeling/moe/linearize.py)."""
import contextlib

from . import get_non_linearized_moes, linearize_moe  # noqa: F401

__all__ = ["linearize_moe", "get_non_linearized_moes", "load_quantizable_moe"]


@contextlib.contextmanager
def load_quantizable_moe(model_cls=None):
    """The reference patches ``from_pretrained`` so that fused experts are split while the checkpoint loads
    (modeling/moe/linearize.py); here the model loads as it is and ``oneshot`` / ``linearize_moe`` split the
    experts afterwards, so nothing is patched."""
    yield
