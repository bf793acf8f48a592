"""Observers that share an NVFP4 global scale (q/k/v, gate/up, ...): who belongs together, lazy observation of
partners, and when the shared statistics may go (behaviour of the reference's observers/fusion.py:17-105).

One ``_FusedSet`` object is shared by the handlers of a fused set.  It holds the members in a fixed order, weak
references to their modules (a partner whose weight has not been observed yet is observed on demand), and the
members that have already asked for their statistics to be dropped; the statistics of the whole set are dropped
when the last member asks, because every member's global scale needs all of them.
"""
from __future__ import annotations

import weakref
from typing import TYPE_CHECKING, Iterable

import torch
from torch.nn import Module

if TYPE_CHECKING:
    from .base import Observer

__all__ = ["FusionHandler"]


class _FusedSet:
    def __init__(self, members: list["FusionHandler"]):
        self.members = members
        self.released: set[int] = set()  # ids of the handlers that are done with the shared statistics

    def release(self, handler: "FusionHandler") -> None:
        self.released.add(id(handler))
        if len(self.released) < len(self.members):
            return
        self.released.clear()
        for member in self.members:
            member.observer.delete_statistics(check_fused=False)


class FusionHandler:
    """Every Observer owns one; it stands alone until ``fuse`` puts it into a set."""

    def __init__(self, observer: "Observer"):
        self.observer = observer
        self._module: weakref.ref | None = None
        self._set: _FusedSet | None = None

    @property
    def is_fused(self) -> bool:
        return self._set is not None and len(self._set.members) > 1

    @property
    def module(self) -> Module | None:
        return self._module() if self._module is not None else None

    @classmethod
    def fuse(cls, observers_and_modules: Iterable[tuple["Observer", Module]]) -> None:
        """Put the observers of the (observer, module) pairs into one set; the modules are only weakly held."""
        members = []
        for observer, module in observers_and_modules:
            handler = observer.fusion_handler
            handler._module = weakref.ref(module)
            members.append(handler)
        shared = _FusedSet(members)
        for handler in members:
            handler._set = shared

    def _members(self) -> list["FusionHandler"]:
        if self._set is None:
            return [self]
        # this handler's own statistics first, as callers expect
        return [self] + [m for m in self._set.members if m is not self]

    def get_fused_statistics(self) -> list[dict[str, torch.Tensor]]:
        """Statistics of this observer and of every partner, observing a partner's weight first if needed."""
        members = self._members()
        for member in members:
            if member.observer.has_statistics:
                continue
            module = member.module
            assert module is not None, "Fused module has been garbage collected before its weight was observed"
            member.observer(module.weight)
        return [member.observer.get_statistics() for member in members]

    def maybe_delete_statistics(self) -> None:
        """This observer no longer needs the statistics: drop them now if it stands alone, else when every
        member of its set has said the same."""
        if self.is_fused:
            self._set.release(self)
        else:
            self.observer.delete_statistics(check_fused=False)
