"""Min-max observers (reference: observers/min_max.py:10-74)."""
import torch

from .base import Observer
from .helpers import lerp

__all__ = ["MemorylessMinMaxObserver", "StaticMinMaxObserver", "MinMaxObserver"]


@Observer.register("memoryless_minmax")
class MemorylessMinMaxObserver(Observer):
    """min/max of the observed value."""


@Observer.register("static_minmax")
class StaticMinMaxObserver(MemorylessMinMaxObserver):
    """min/max over everything observed so far."""

    def update_statistics(self, min_vals, max_vals):
        if hasattr(self, "min_vals"):
            min_vals = torch.min(min_vals, self.min_vals)
            max_vals = torch.max(max_vals, self.max_vals)
        self.min_vals, self.max_vals = min_vals, max_vals


@Observer.register("minmax")
class MinMaxObserver(Observer):
    """exponential moving average of min/max."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.avg_constant = self.args.observer_kwargs.get("averaging_constant", 0.01)

    def update_statistics(self, min_vals, max_vals):
        if hasattr(self, "min_vals") and self.avg_constant != 1.0:
            min_vals = lerp(self.min_vals, min_vals, self.avg_constant)
            max_vals = lerp(self.max_vals, max_vals, self.avg_constant)
        self.min_vals, self.max_vals = min_vals, max_vals
