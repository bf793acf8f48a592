"""``llmcompressor``: the reference's import root, served by ``llmcompressor_amd``.

``from llmcompressor import oneshot, model_free_ptq``, ``from llmcompressor.modifiers.gptq import GPTQModifier``,
``from llmcompressor.modifiers.quantization import GPTQModifier, QuantizationModifier`` and the deprecated
``llmcompressor.modifiers.quantization.gptq`` (reference: src/llmcompressor/__init__.py:23-29,
modifiers/quantization/__init__.py, modifiers/quantization/gptq/__init__.py) resolve to the very same module
objects as their ``llmcompressor_amd`` counterparts: a finder on ``sys.meta_path`` maps every
``llmcompressor.<path>`` to ``llmcompressor_amd.<path>``, so registries, the active session and class identities
are shared whichever root a caller imports from.  Nothing is computed here.
"""
from __future__ import annotations

import importlib
import importlib.abc
import importlib.util
import sys

import llmcompressor_amd as _target

_ALIAS, _REAL = __name__, _target.__name__


class _AliasLoader(importlib.abc.Loader):
    def __init__(self, real_name: str):
        self._real_name = real_name

    def create_module(self, spec):
        return importlib.import_module(self._real_name)  # the same module object under a second name

    def exec_module(self, module):
        pass


class _AliasFinder(importlib.abc.MetaPathFinder):
    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith(_ALIAS + "."):
            return None
        real_name = _REAL + fullname[len(_ALIAS):]
        try:
            real_spec = importlib.util.find_spec(real_name)
        except ModuleNotFoundError:
            return None
        if real_spec is None:
            return None
        spec = importlib.util.spec_from_loader(fullname, _AliasLoader(real_name),
                                               is_package=real_spec.submodule_search_locations is not None)
        return spec


if not any(isinstance(f, _AliasFinder) for f in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())

__version__ = _target.__version__
version = __version__
__all__ = ["__version__", "version", "oneshot", "model_free_ptq", "active_session", "create_session",
           "reset_session", "callbacks"]


def __getattr__(name):
    if name in ("oneshot", "Oneshot", "model_free_ptq"):
        return getattr(importlib.import_module(_REAL + ".entrypoints"), name)
    if name in ("active_session", "create_session", "reset_session", "callbacks"):
        core = importlib.import_module(_REAL + ".core")
        if name == "callbacks":
            return core.LifecycleCallbacks
        return getattr(core, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
