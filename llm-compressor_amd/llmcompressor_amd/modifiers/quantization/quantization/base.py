"""QuantizationModifier: round-to-nearest PTQ (reference: modifiers/quantization/quantization/base.py:24-114)."""
from __future__ import annotations

import torch

from ....core import Event, State
from ....observers import ACTIVATION_OBS
from ....quantization import is_module_quantized
from ...modifier import Modifier
from ..calibration import observe, update_qparams
from .mixin import QuantizationMixin

__all__ = ["QuantizationModifier"]


class QuantizationModifier(Modifier, QuantizationMixin):
    """Weights (and optionally static activations) are observed and their qparams stored; the
    checkpoint writer then packs them.  Lifecycle as in the reference: on_initialize applies the
    config, calibration start attaches observers/hooks, every sequential epoch end observes the
    weights of the finished modules, calibration end freezes."""

    def on_initialize(self, state: State, **kwargs) -> bool:
        if not QuantizationMixin.has_config(self):
            raise ValueError("QuantizationModifier requires that quantization fields be specified")
        QuantizationMixin.initialize_quantization(self, state.model)
        return True

    def on_calibration_start(self, state: State, event: Event, **kwargs):
        QuantizationMixin.start_calibration(self, state.model)

    def on_sequential_epoch_end(self, state: State, event: Event, modules: list[torch.nn.Module] = (), **kwargs):
        modules = [m for m in modules if is_module_quantized(m)]
        self.sync_obs_act_stats(modules)
        update_qparams(modules, ACTIVATION_OBS)
        observe(modules, "weight")
        update_qparams(modules, "weight")

    def on_calibration_end(self, state: State, event: Event, **kwargs):
        QuantizationMixin.end_calibration(self, state.model)

    def on_finalize(self, state: State, **kwargs) -> bool:
        return True
