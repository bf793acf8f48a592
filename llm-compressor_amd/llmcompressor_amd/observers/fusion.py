"""Fusion bookkeeping for observers that share an NVFP4 global scale (reference: observers/fusion.py:17-105)."""
from __future__ import annotations

from typing import TYPE_CHECKING, Iterable
from weakref import ref

import torch
from torch.nn import Module

if TYPE_CHECKING:
    from .base import Observer

__all__ = ["FusionHandler"]

_msg = "Fused module has been garbage collected before its weight was observed"


class FusionHandler:
    def __init__(self, observer: "Observer"):
        self._observer = observer
        self._module_ref: ref[Module] | None = None
        self._group: list[FusionHandler] = []
        self._deletion_called = False

    @property
    def is_fused(self) -> bool:
        return len(self._group) > 0

    @property
    def module(self) -> Module | None:
        return None if self._module_ref is None else self._module_ref()

    @classmethod
    def fuse(cls, observers_and_modules: Iterable[tuple["Observer", Module]]) -> None:
        handlers = []
        for obs, mod in list(observers_and_modules):
            obs.fusion_handler._module_ref = ref(mod)
            handlers.append(obs.fusion_handler)
        for h in handlers:
            h._group = [o for o in handlers if o is not h]

    def get_fused_statistics(self) -> list[dict[str, torch.Tensor]]:
        handlers = [self] + self._group
        for h in handlers:
            obs = h._observer
            if not obs.has_statistics:
                mod = h.module
                assert mod is not None, _msg
                obs(mod.weight)
        return [h._observer.get_statistics() for h in handlers]

    def maybe_delete_statistics(self) -> None:
        if not self.is_fused:
            self._delete(self._observer)
            return
        self._deletion_called = True
        if all(h._deletion_called for h in self._group):
            self._deletion_called = False
            for h in self._group:
                h._deletion_called = False
                self._delete(h._observer)
            self._delete(self._observer)

    @staticmethod
    def _delete(observer: "Observer") -> None:
        observer.delete_statistics(check_fused=False)
