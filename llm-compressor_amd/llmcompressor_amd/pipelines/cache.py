"""Cache of the intermediate values (activations) that flow between the sequential targets of a model
(reference: pipelines/cache.py:16-300).

Same interface as the reference's ``IntermediatesCache`` -- ``empty`` / ``from_dataloader``, ``fetch``,
``update``, ``delete``, ``append``, ``size``, ``iter`` / ``iter_prefetch`` -- with one difference in the
default: ``offload_device=None``, i.e. the values stay where they were produced.  A full calibration
set of hidden states (256 x 2048 x 4096 bf16 = 4 GiB) is small next to 288 GB of HBM, so the two
host-device copies per batch per layer that the CPU-offloading default implies are simply not made.
Passing ``offload_device="cpu"`` gives the reference's behaviour.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, fields, is_dataclass
from typing import Any, Dict, Generator, List, Optional

import torch

__all__ = ["IntermediateValue", "IntermediatesCache"]


@dataclass
class IntermediateValue:
    """A cached value: an (offloaded) tensor, a primitive, or a container of IntermediateValues;
    ``device`` is where a tensor goes back to when fetched."""

    value: Any
    device: Optional[torch.device]


class IntermediatesCache:
    batch_intermediates: List[Dict[str, IntermediateValue]]
    offload_device: Optional[torch.device]

    def __init__(self, batch_intermediates: Optional[List[Dict[str, IntermediateValue]]] = None,
                 offload_device: Optional[torch.device | str] = None):
        self.batch_intermediates = batch_intermediates or []
        self.offload_device = None if offload_device is None else torch.device(offload_device)

    # ---- construction
    @classmethod
    def empty(cls, num_batches: int, offload_device: Optional[torch.device | str] = None) -> "IntermediatesCache":
        return cls([{} for _ in range(num_batches)], offload_device)

    @classmethod
    def from_dataloader(cls, dataloader, model_device: torch.device | str = torch.device("cpu"),
                        offload_device: Optional[torch.device | str] = None) -> "IntermediatesCache":
        """One entry per batch of the dataloader; tensors are fetched onto ``model_device``."""
        model_device = torch.device(model_device)
        off = None if offload_device is None else torch.device(offload_device)
        batches = []
        for batch in dataloader:
            if not isinstance(batch, dict):
                batch = {"input_ids": batch}
            batches.append({k: cls._offload_value(v, off, model_device) for k, v in batch.items()})
        return cls(batches, off)

    # ---- access
    def fetch(self, batch_index: int, input_names: Optional[List[str]] = None) -> Dict[str, Any]:
        inter = self.batch_intermediates[batch_index]
        return {k: self._onload_value(v) for k, v in inter.items() if input_names is None or k in input_names}

    def update(self, batch_index: int, values: Dict[str, Any]):
        self.batch_intermediates[batch_index].update(
            {k: self._offload_value(v, self.offload_device) for k, v in values.items()})

    def delete(self, batch_index: int, consumed_names: Optional[List[str]] = None):
        inter = self.batch_intermediates[batch_index]
        for name in list(inter.keys()) if consumed_names is None else consumed_names:
            del inter[name]

    def append(self, values: Dict[str, Any]):
        self.batch_intermediates.append({})
        self.update(len(self.batch_intermediates) - 1, values)

    def size(self) -> Dict[torch.device, int]:
        """Bytes held, per device."""
        sizes: Dict[torch.device, int] = {}
        seen = set()

        def walk(iv: IntermediateValue):
            v = iv.value
            if isinstance(v, torch.Tensor):
                key = (v.device, v.data_ptr(), v.numel())
                if key not in seen:
                    seen.add(key)
                    sizes[v.device] = sizes.get(v.device, 0) + v.numel() * v.element_size()
            elif isinstance(v, (list, tuple)):
                for x in v:
                    walk(x)
            elif isinstance(v, dict):
                for x in v.values():
                    walk(x)
            elif is_dataclass(v) and not isinstance(v, type):
                for f in fields(v):
                    walk(getattr(v, f.name))

        for inter in self.batch_intermediates:
            for iv in inter.values():
                walk(iv)
        return sizes

    def iter(self, input_names: Optional[List[str]] = None) -> Generator[Dict[str, Any], None, None]:
        for i in range(len(self.batch_intermediates)):
            yield self.fetch(i, input_names)

    def iter_prefetch(self, input_names: Optional[List[str]] = None) -> Generator[Dict[str, Any], None, None]:
        """Same batches as ``iter``.  With device-resident values there is nothing to prefetch; with an
        offload device the next batch's copy is issued (non-blocking) before the current one is yielded."""
        n = len(self.batch_intermediates)
        if n == 0:
            return
        nxt = self.fetch(0, input_names)
        for i in range(n):
            cur = nxt
            if i + 1 < n:
                nxt = self.fetch(i + 1, input_names)
            yield cur

    def __iter__(self):
        yield from self.iter()

    def __len__(self) -> int:
        return len(self.batch_intermediates)

    # ---- recursion over containers
    @classmethod
    def _offload_value(cls, value: Any, offload_device: Optional[torch.device],
                       onload_device: Optional[torch.device] = None) -> IntermediateValue:
        if isinstance(value, torch.Tensor):
            target = onload_device if onload_device is not None else value.device
            keep_on = target if offload_device is None else offload_device
            return IntermediateValue(value if value.device == keep_on else value.to(keep_on), target)
        if isinstance(value, tuple):
            return IntermediateValue(tuple(cls._offload_value(v, offload_device, onload_device) for v in value), None)
        if isinstance(value, list):
            return IntermediateValue([cls._offload_value(v, offload_device, onload_device) for v in value], None)
        if isinstance(value, dict):
            return IntermediateValue({k: cls._offload_value(v, offload_device, onload_device)
                                      for k, v in value.items()}, None)
        if is_dataclass(value) and not isinstance(value, type):
            held = copy.copy(value)  # the caller's object keeps its own fields
            for f in fields(value):
                setattr(held, f.name, cls._offload_value(getattr(value, f.name), offload_device, onload_device))
            return IntermediateValue(held, None)
        return IntermediateValue(value, None)  # primitives, None, ...

    @classmethod
    def _onload_value(cls, iv: IntermediateValue) -> Any:
        v = iv.value
        if isinstance(v, torch.Tensor):
            return v if iv.device is None or v.device == iv.device else v.to(iv.device, non_blocking=True)
        if isinstance(v, tuple):
            return tuple(cls._onload_value(x) for x in v)
        if isinstance(v, list):
            return [cls._onload_value(x) for x in v]
        if isinstance(v, dict):
            return {k: cls._onload_value(x) for k, x in v.items()}
        if is_dataclass(v) and not isinstance(v, type):
            out = type(v)(**{f.name: cls._onload_value(getattr(v, f.name)) for f in fields(v)})
            return out
        return v
