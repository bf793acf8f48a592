"""Where a model that arrives on the host is computed on.

The reference's pipelines call ``set_onload_device(model, get_main_device())`` first
(pipelines/sequential/pipeline.py:85-87, pipelines/data_free/pipeline.py:34-35): a model loaded with
``from_pretrained`` sits in host memory, every module is brought to the accelerator when it runs and sent back
afterwards.  One MI355X holds 288 GB, so a model that fits is moved to the GPU once and stays there; only a model
larger than that is calibrated with one decoder layer on the GPU at a time (sequential pipeline).
"""
from __future__ import annotations

import logging
from typing import Optional

import torch

logger = logging.getLogger("llmcompressor_amd")

__all__ = ["get_main_device", "model_bytes", "place_model", "RESIDENT_FRACTION"]

# share of the GPU's free memory a model may take and still be kept resident; the rest is for the calibration
# activations, the Hessians of a layer (0.8 GB for a 14336-wide Linear) and the quantisation workspaces
RESIDENT_FRACTION = 0.6


def get_main_device() -> torch.device:
    """The GPU this process computes on, or the host when there is none (reference: utils/dev.py:157-173)."""
    if torch.cuda.is_available():
        return torch.device("cuda", torch.cuda.current_device())
    logger.warning("No accelerator available! Compressing model on CPU instead")
    return torch.device("cpu")


def model_bytes(model: torch.nn.Module) -> int:
    seen, total = set(), 0
    for t in list(model.parameters()) + list(model.buffers()):
        if t.data_ptr() in seen:
            continue
        seen.add(t.data_ptr())
        total += t.numel() * t.element_size()
    return total


def place_model(model: torch.nn.Module) -> Optional[torch.device]:
    """Move a host-resident model to the GPU if it fits and return None; return the GPU to onload layers to if it
    does not fit.  A model that already has a parameter on a GPU (or none at all, or meta tensors) is left as its
    caller placed it."""
    params = list(model.parameters())
    if not params or any(p.device.type != "cpu" for p in params):
        return None
    device = get_main_device()
    if device.type == "cpu":
        return None
    free, _total = torch.cuda.mem_get_info(device)
    need = model_bytes(model)
    if need <= RESIDENT_FRACTION * free:
        logger.info(f"moving the model ({need / 2**30:.1f} GiB) to {device} for calibration; it stays there")
        model.to(device)
        return None
    logger.info(f"the model ({need / 2**30:.1f} GiB) does not fit beside its calibration state in "
                f"{free / 2**30:.1f} GiB of free GPU memory: one layer at a time is brought to {device}")
    return device
