"""Calibration pipelines (reference: src/llmcompressor/pipelines/).

* ``sequential``: one decoder layer at a time, two passes per layer -- calibrate with hooks, fire
  ``sequential_epoch_end`` (observers + quantize_weight), then propagate through the now-quantised
  layer with hooks disabled (pipelines/sequential/pipeline.py:136-181).  The reference finds the
  layer boundaries by tracing the model with torch.fx; here the boundaries are the model's list of
  decoder layers, which is the same partition for decoder-only transformers.  Activations stay
  resident in HBM between layers instead of being offloaded to the host.
* ``datafree``: calibration_start -> sequential_epoch_end(all modules) -> calibration_end.
* ``basic``: one pass over the data through the whole model, then the epoch-end events.
* ``independent``: one inferred pipeline per modifier.
"""
from __future__ import annotations

import contextlib
from typing import Dict, List, Optional

import torch

from ..core import LifecycleCallbacks, active_session
from ..modifiers.utils.hooks import HooksMixin
from ..quantization import disable_quantization, enable_quantization

__all__ = ["CalibrationPipeline", "SequentialPipeline", "DataFreePipeline", "BasicPipeline", "IndependentPipeline",
           "calibration_forward_context", "DisableQuantization", "find_decoder_layers"]


@contextlib.contextmanager
def calibration_forward_context(model: torch.nn.Module):
    """no_grad, eval mode, no KV cache (reference: utils/helpers.py:120-137)."""
    was_training = model.training
    cfg = getattr(model, "config", None)
    had = getattr(cfg, "use_cache", None)
    model.eval()
    if cfg is not None and had is not None:
        cfg.use_cache = False
    try:
        with torch.no_grad():
            yield
    finally:
        if cfg is not None and had is not None:
            cfg.use_cache = had
        model.train(was_training)


@contextlib.contextmanager
def DisableQuantization(model: torch.nn.Module):
    model.apply(disable_quantization)
    try:
        yield
    finally:
        model.apply(enable_quantization)


class CalibrationPipeline:
    _registry: Dict[str, type] = {}

    @classmethod
    def register(cls, name):
        def deco(klass):
            CalibrationPipeline._registry[name] = klass
            return klass

        return deco

    @classmethod
    def load_from_registry(cls, name):
        return CalibrationPipeline._registry[name]()

    @classmethod
    def from_modifiers(cls, modifiers: List, user: Optional[str] = None) -> "CalibrationPipeline":
        inferred = "sequential" if any(m.requires_calibration_data for m in modifiers) else "datafree"
        if user is not None and user != inferred and user != "independent":
            return cls.load_from_registry(user)
        if user == "independent":
            return cls.load_from_registry("independent")
        return cls.load_from_registry(inferred)

    def __call__(self, model, dataloader, dataset_args=None):
        raise NotImplementedError()


def find_decoder_layers(model: torch.nn.Module, sequential_targets=None) -> List[torch.nn.Module]:
    """The modules that form the sequential partition: explicit class names, else the model's own
    ``_no_split_modules`` (what the reference infers for transformers models), else the longest ModuleList
    that is not nested inside an element of another one (an experts list inside a decoder layer is not the
    layer list)."""
    if sequential_targets:
        names = [sequential_targets] if isinstance(sequential_targets, str) else list(sequential_targets)
        layers = [m for m in model.modules() if m.__class__.__name__ in names]
        if layers:
            return layers
    no_split = getattr(model, "_no_split_modules", None)
    if no_split:
        layers = [m for m in model.modules() if m.__class__.__name__ in set(no_split)]
        # nested matches (a no-split block inside another) would run twice: keep the outermost
        inner = {id(x) for l in layers for x in l.modules() if x is not l}
        layers = [l for l in layers if id(l) not in inner]
        if layers:
            return layers
    lists = [m for m in model.modules() if isinstance(m, torch.nn.ModuleList) and len(m) > 0]
    nested = set()
    for outer in lists:
        for element in outer:
            nested.update(id(x) for x in element.modules() if isinstance(x, torch.nn.ModuleList))
    best = None
    for m in lists:
        if id(m) not in nested and (best is None or len(m) > len(best)):
            best = m
    if best is None:
        raise ValueError("could not infer sequential targets: the model has no ModuleList of layers")
    return list(best)


from .cache import IntermediatesCache  # noqa: E402


class _StopForward(Exception):
    pass


@CalibrationPipeline.register("sequential")
class SequentialPipeline(CalibrationPipeline):
    def __call__(self, model, dataloader, dataset_args=None):
        targets = getattr(dataset_args, "sequential_targets", None) if dataset_args is not None else None
        layers = find_decoder_layers(model, targets)
        device = next(model.parameters()).device
        LifecycleCallbacks.calibration_start()
        with calibration_forward_context(model), DisableQuantization(model):
            # capture the first layer's inputs for every batch (activations stay on the device)
            captured = []

            def grab(_module, args, kwargs):
                captured.append((args, kwargs))
                raise _StopForward()

            handle = layers[0].register_forward_pre_hook(grab, with_kwargs=True)
            try:
                for batch in dataloader:
                    batch = _to_device(batch, device)
                    try:
                        model(**batch) if isinstance(batch, dict) else model(batch)
                    except _StopForward:
                        pass
            finally:
                handle.remove()
            # the activations between layers live in a device-resident cache (no CPU offload)
            offload = getattr(dataset_args, "sequential_offload_device", None) if dataset_args is not None else None
            cache = IntermediatesCache.empty(len(captured), offload_device=offload)
            for i, (args, kwargs) in enumerate(captured):
                cache.update(i, {"args": tuple(args), "kwargs": dict(kwargs)})
            del captured
            for idx, layer in enumerate(layers):
                # pass 1: calibrate (hooks fire: Hessians / activation observers)
                for inputs in cache.iter_prefetch():
                    layer(*inputs["args"], **inputs["kwargs"])
                LifecycleCallbacks.sequential_epoch_end(modules=list(layer.modules()))
                # pass 2: propagate through the compressed layer without triggering hooks
                with HooksMixin.disable_hooks():
                    for i in range(len(cache)):
                        inputs = cache.fetch(i)
                        out = layer(*inputs["args"], **inputs["kwargs"])
                        hidden = out[0] if isinstance(out, (tuple, list)) else out
                        cache.update(i, {"args": (hidden,) + tuple(inputs["args"][1:])})
            # modules outside the layer list (e.g. lm_head) that modifiers may target
            rest = [m for m in model.modules() if not any(m is x for l in layers for x in l.modules())]
            LifecycleCallbacks.sequential_epoch_end(modules=rest)
        LifecycleCallbacks.calibration_end()


@CalibrationPipeline.register("datafree")
class DataFreePipeline(CalibrationPipeline):
    def __call__(self, model, dataloader=None, dataset_args=None):
        LifecycleCallbacks.calibration_start()
        LifecycleCallbacks.sequential_epoch_end(modules=list(model.modules()))
        LifecycleCallbacks.calibration_end()


@CalibrationPipeline.register("basic")
class BasicPipeline(CalibrationPipeline):
    def __call__(self, model, dataloader, dataset_args=None):
        device = next(model.parameters()).device
        LifecycleCallbacks.calibration_start()
        with calibration_forward_context(model):
            for batch in dataloader:
                batch = _to_device(batch, device)
                model(**batch) if isinstance(batch, dict) else model(batch)
            LifecycleCallbacks.sequential_epoch_end(modules=list(model.modules()))
        LifecycleCallbacks.calibration_end()


@CalibrationPipeline.register("independent")
class IndependentPipeline(CalibrationPipeline):
    def __call__(self, model, dataloader, dataset_args=None):
        session = active_session()
        mods = session.get_modifiers()
        recipe = session.lifecycle.recipe
        try:
            for m in mods:
                recipe.modifiers = [m]
                pipeline = CalibrationPipeline.from_modifiers([m])
                pipeline(model, dataloader, dataset_args)
        finally:
            recipe.modifiers = mods


def _to_device(batch, device):
    if isinstance(batch, dict):
        return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in batch.items()}
    if torch.is_tensor(batch):
        return batch.to(device)
    return batch
