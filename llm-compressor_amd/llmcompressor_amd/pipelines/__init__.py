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
import logging
from typing import Dict, List, Optional

import torch

from ..core import LifecycleCallbacks, active_session
from ..modifiers.utils.hooks import HooksMixin
from ..quantization import disable_quantization, enable_quantization

logger = logging.getLogger("llmcompressor_amd")

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
        if layers and _is_chain(model, layers):
            return layers
        if layers:
            # The reference cuts the traced graph at any module class (attention and each expert of one decoder
            # layer as separate subgraphs, to bound the Hessians held at once); this pipeline feeds each target's
            # output to the next one, which only whole layers of one list allow.  A decoder layer's Hessians fit
            # the GPU, so the layer partition is used instead of failing.
            logger.warning(f"sequential_targets {names} are not the elements of one layer list; calibrating by "
                           "decoder layer instead")
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


def _is_chain(model: torch.nn.Module, layers: List[torch.nn.Module]) -> bool:
    """Are `layers` exactly the elements of one ModuleList (so that each one's output is the next one's input)?"""
    ids = {id(l) for l in layers}
    for m in model.modules():
        if isinstance(m, torch.nn.ModuleList) and len(m) == len(layers) and all(id(x) in ids for x in m):
            return True
    return False


from .cache import IntermediatesCache  # noqa: E402


class _StopForward(Exception):
    pass


@CalibrationPipeline.register("sequential")
class SequentialPipeline(CalibrationPipeline):
    def __call__(self, model, dataloader, dataset_args=None):
        targets = getattr(dataset_args, "sequential_targets", None) if dataset_args is not None else None
        layers = find_decoder_layers(model, targets)
        # a model too large to stay on the GPU: what surrounds the layers (embeddings, final norm, head) is
        # brought over for the whole run, each layer for its two passes, and everything returns to the host
        onload = getattr(dataset_args, "onload_device", None) if dataset_args is not None else None
        home = next(model.parameters()).device
        device = onload if onload is not None else home
        inside = {id(x) for l in layers for x in l.modules()}
        rest = [m for m in model.modules() if id(m) not in inside]
        if onload is not None:
            for m in rest:
                m._apply(lambda t: t.to(onload), recurse=False)
        try:
            self._run(model, dataloader, dataset_args, layers, rest, device, onload, home)
        finally:
            if onload is not None:
                for m in model.modules():
                    m._apply(lambda t: t.to(home), recurse=False)

    def _run(self, model, dataloader, dataset_args, layers, rest, device, onload, home):
        LifecycleCallbacks.calibration_start()
        with calibration_forward_context(model), DisableQuantization(model):
            # capture the first layer's inputs for every batch (activations stay on the device)
            captured = []

            def grab(_module, args, kwargs):
                captured.append((args, kwargs))
                raise _StopForward()

            before = set()  # modules that run ahead of the first layer (their hooks fire in this capture pass)
            trackers = [m.register_forward_pre_hook(lambda mod, args: before.add(id(mod))) for m in rest]
            handle = layers[0].register_forward_pre_hook(grab, with_kwargs=True)
            try:
                for batch in dataloader:
                    batch = _to_device(batch, device)
                    try:
                        model(**batch) if isinstance(batch, dict) else model(batch)
                    except _StopForward:
                        pass
                    for t in trackers:
                        t.remove()
                    trackers = []
            finally:
                handle.remove()
                for t in trackers:
                    t.remove()
            # the activations between layers live in a device-resident cache (no CPU offload)
            offload = getattr(dataset_args, "sequential_offload_device", None) if dataset_args is not None else None
            cache = IntermediatesCache.empty(len(captured), offload_device=offload)
            for i, (args, kwargs) in enumerate(captured):
                cache.update(i, {"args": tuple(args), "kwargs": dict(kwargs)})
            del captured
            returns_tuple = False
            # reference: pipelines/sequential/pipeline.py:155-176 -- with ``propagate_error=False`` the next layer
            # is fed what the calibration pass produced (the outputs of the layer before it was compressed) and
            # the second pass is not run: half the forwards
            propagate = getattr(dataset_args, "propagate_error", True) if dataset_args is not None else True
            # reference: ``sequential_targets_per_subgraph`` (pipelines/sequential/helpers.py) -- that many
            # consecutive layers are calibrated together, each on what the uncompressed layers before it in the
            # group produce, and compressed by one epoch-end event
            per = getattr(dataset_args, "sequential_targets_per_subgraph", 1) if dataset_args is not None else 1
            per = max(1, int(per or 1))

            def through(group, inputs):
                """The group's layers one after the other on one batch; returns the arguments for what follows."""
                nonlocal returns_tuple
                args = tuple(inputs["args"])
                for member in group:
                    out = member(*args, **inputs["kwargs"])
                    returns_tuple = isinstance(out, (tuple, list))
                    args = ((out[0] if returns_tuple else out),) + args[1:]
                return args

            for start in range(0, len(layers), per):
                group = layers[start:start + per]
                if onload is not None:
                    for layer in group:
                        layer.to(onload)
                # pass 1: calibrate (hooks fire: Hessians / activation observers)
                if propagate:
                    for inputs in cache.iter_prefetch():
                        through(group, inputs)
                else:
                    for i in range(len(cache)):
                        cache.update(i, {"args": through(group, cache.fetch(i))})
                LifecycleCallbacks.sequential_epoch_end(modules=[m for layer in group for m in layer.modules()])
                # pass 2: propagate through the compressed layers without triggering hooks
                if propagate:
                    with HooksMixin.disable_hooks():
                        for i in range(len(cache)):
                            cache.update(i, {"args": through(group, cache.fetch(i))})
                if onload is not None:
                    for layer in group:
                        layer.to(home)
            # what follows the last layer (final norm, lm_head): the reference's last traced subgraph holds it
            # (pipelines/sequential/pipeline.py:136-181), so a module there that a modifier hooked is calibrated too
            tail = [m for m in rest if id(m) not in before and _has_calibration_hooks(m)]
            if tail:
                _calibrate_tail(model, layers, tail, dataloader, cache, device, returns_tuple)
            LifecycleCallbacks.sequential_epoch_end(modules=rest)
        LifecycleCallbacks.calibration_end()


def _has_calibration_hooks(module: torch.nn.Module) -> bool:
    """Did a modifier register a forward (pre-)hook on this very module?"""
    return bool(module._forward_hooks) or bool(module._forward_pre_hooks)


def _calibrate_tail(model, layers, tail, dataloader, cache, device, returns_tuple: bool) -> None:
    """Run what follows the last sequential layer on every cached hidden state, with the hooks of `tail` on.

    The model is called on the original batches while every sequential layer is short-circuited: the last one
    returns the cached output of the propagation pass, the others hand their input through.  What precedes
    the layers (embeddings, rotary tables) is recomputed, which is cheap; its hooks fired in the capture pass
    already, so only the handles registered on the `tail` modules are kept enabled."""
    keep = set()
    for m in tail:
        keep.update(_handles_of(m))
    current = {}

    def hand_through(*args, **kwargs):
        hidden_states = args[0] if args else kwargs["hidden_states"]
        return (hidden_states,) if returns_tuple else hidden_states

    def cached_output(*args, **kwargs):
        return (current["hidden"],) if returns_tuple else current["hidden"]

    missing = object()
    patched = []  # (layer, the instance-level forward it carried before, or `missing`)
    seen = 0
    try:
        for layer in layers[:-1]:
            patched.append((layer, vars(layer).get("forward", missing)))
            layer.forward = hand_through
        patched.append((layers[-1], vars(layers[-1]).get("forward", missing)))
        layers[-1].forward = cached_output
        with HooksMixin.disable_hooks(keep=keep):
            for i, batch in enumerate(dataloader):
                if i >= len(cache):
                    break
                current["hidden"] = cache.fetch(i)["args"][0]
                batch = _to_device(batch, device)
                model(**batch) if isinstance(batch, dict) else model(batch)
                seen += 1
    finally:
        for layer, previous in patched:
            if previous is missing:
                del layer.forward  # back to the class's method
            else:
                layer.forward = previous  # a wrapper assigned on the instance (e.g. an offloading hook) stays in place
    if seen < len(cache):
        # a one-shot iterable is exhausted after the first pass: the modules after the last layer would be left
        # with fewer samples than the layers (none at all, a zero Hessian), which must not pass silently
        raise RuntimeError(
            f"the calibration data yielded {seen} batches on the pass for the modules after the last layer, "
            f"{len(cache)} on the first pass; pass a re-iterable dataloader (a list or a DataLoader)")


def _handles_of(module: torch.nn.Module):
    """The RemovableHandle objects of the hooks registered on `module`, as HooksMixin keeps them."""
    from torch.utils.hooks import RemovableHandle

    ids = set(module._forward_hooks) | set(module._forward_pre_hooks)
    return {h for h in HooksMixin._ALL_HANDLES if isinstance(h, RemovableHandle) and h.id in ids}


@CalibrationPipeline.register("datafree")
class DataFreePipeline(CalibrationPipeline):
    def __call__(self, model, dataloader=None, dataset_args=None):
        _refuse_layerwise(dataset_args, "datafree")
        LifecycleCallbacks.calibration_start()
        LifecycleCallbacks.sequential_epoch_end(modules=list(model.modules()))
        LifecycleCallbacks.calibration_end()


@CalibrationPipeline.register("basic")
class BasicPipeline(CalibrationPipeline):
    def __call__(self, model, dataloader, dataset_args=None):
        _refuse_layerwise(dataset_args, "basic")
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


def _refuse_layerwise(dataset_args, name: str):
    if dataset_args is not None and getattr(dataset_args, "onload_device", None) is not None:
        raise RuntimeError(
            f"the model does not fit in GPU memory and the {name!r} pipeline works on the whole model at once; "
            "quantise the checkpoint shard by shard with `model_free_ptq`, or use a recipe that calibrates "
            "through the sequential pipeline")


def _to_device(batch, device):
    if isinstance(batch, dict):
        return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in batch.items()}
    if torch.is_tensor(batch):
        return batch.to(device)
    return batch
