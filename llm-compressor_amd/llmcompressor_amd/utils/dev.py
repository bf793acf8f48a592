"""Loading and placement helpers the reference's examples import from ``llmcompressor.utils``
(reference: utils/dev.py:36-52, 157-200).

The reference needs them because it keeps a model in host memory behind offloading hooks and linearises fused MoE
experts while the checkpoint loads.  Here a model is loaded as transformers loads it, ``oneshot`` linearises fused
experts itself and computes on the GPU (``pipelines/onload.py``), so ``load_context`` only has to exist and
``dispatch_for_generation`` is a move to the GPU.
"""
from __future__ import annotations

import contextlib

import torch

from ..pipelines.onload import get_main_device

__all__ = ["load_context", "dispatch_for_generation", "get_main_device"]


@contextlib.contextmanager
def load_context(model_cls=None):
    """``with load_context(): model = AutoModelForCausalLM.from_pretrained(...)`` loads the model to host memory
    as usual; nothing is patched."""
    yield


def dispatch_for_generation(model: torch.nn.Module, *args, **kwargs) -> torch.nn.Module:
    """Place the model for ``generate`` after ``oneshot``: on the GPU (it fits one MI355X or it would not have
    been kept there), on the host when there is no GPU."""
    device = get_main_device()
    if device.type != "cpu" and any(p.device != device for p in model.parameters()):
        model.to(device)
    return model
