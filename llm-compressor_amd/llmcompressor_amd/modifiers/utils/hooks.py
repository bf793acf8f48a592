"""Hook registration with a global disable switch (reference: modifiers/utils/hooks.py:19-133)."""
from __future__ import annotations

import contextlib
import weakref
from functools import wraps
from typing import Any, Callable, ClassVar

import torch
from pydantic import BaseModel, PrivateAttr
from torch.utils.hooks import RemovableHandle

__all__ = ["HooksMixin", "hook_is_inert"]


def hook_is_inert(fn) -> bool:
    """True for a hook function registered through ``HooksMixin.register_hook`` that is switched off right now
    (``disable_hooks`` is active and its handle is not among the kept ones): calling it would return at once."""
    handle = getattr(fn, "_llmc_handle", None)
    if handle is None:
        return False
    handle = handle()
    return handle is not None and HooksMixin._HOOKS_DISABLED and handle not in HooksMixin._HOOKS_KEEP_ENABLED


class HooksMixin(BaseModel):
    _HOOKS_DISABLED: ClassVar[bool] = False
    _HOOKS_KEEP_ENABLED: ClassVar[set] = set()
    # every handle a modifier still refers to (for `keep` by module); weak, so that a handle removed directly with
    # handle.remove() and dropped by its modifier does not stay alive here
    _ALL_HANDLES: ClassVar[weakref.WeakSet] = weakref.WeakSet()

    _hooks: set = PrivateAttr(default_factory=set)

    @classmethod
    @contextlib.contextmanager
    def disable_hooks(cls, keep: set = frozenset()):
        """Disable all hooks across all modifiers, except the handles in ``keep``."""
        try:
            HooksMixin._HOOKS_DISABLED = True
            HooksMixin._HOOKS_KEEP_ENABLED |= set(keep)
            yield
        finally:
            HooksMixin._HOOKS_DISABLED = False
            HooksMixin._HOOKS_KEEP_ENABLED -= set(keep)

    def register_hook(self, target: torch.nn.Module | torch.nn.Parameter, hook: Callable[[Any], Any], hook_type: str,
                      **kwargs) -> RemovableHandle:
        handle = None

        @wraps(hook)
        def wrapped_hook(*args, **kw):
            if HooksMixin._HOOKS_DISABLED and handle not in HooksMixin._HOOKS_KEEP_ENABLED:
                return
            return hook(*args, **kw)

        name = f"register_{hook_type}_hook" if hook_type else "register_hook"
        register = getattr(target, name)
        handle = register(wrapped_hook, **kwargs)
        wrapped_hook._llmc_handle = weakref.ref(handle)
        self._hooks.add(handle)
        HooksMixin._ALL_HANDLES.add(handle)
        return handle

    def remove_hooks(self, handles: set | None = None):
        if handles is None:
            handles = self._hooks
        for h in list(handles):
            h.remove()
        for h in list(handles):
            HooksMixin._ALL_HANDLES.discard(h)
        self._hooks -= set(handles)
