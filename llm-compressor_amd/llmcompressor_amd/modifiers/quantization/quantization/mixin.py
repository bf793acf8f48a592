"""QuantizationMixin (reference: modifiers/quantization/quantization/mixin.py:56-500)."""
from __future__ import annotations

from typing import Any, Iterator

import torch
from pydantic import Field, PrivateAttr, field_validator, model_validator

from ....observers.helpers import fuse_weight_observers
from ....quantization import (
    DynamicType,
    QuantizationArgs,
    QuantizationConfig,
    QuantizationScheme,
    QuantizationStatus,
    apply_quantization_config,
    disable_quantization,
    enable_quantization,
    is_preset_scheme,
    match_named_modules,
    preset_name_to_scheme,
)
from ...utils.hooks import HooksMixin
from ..calibration import (
    apply_calibration_status,
    calibrate_input_hook,
    calibrate_key_hook,
    calibrate_output_hook,
    calibrate_value_hook,
    freeze_module_quantization,
    initialize_observer,
    reset_quantization_status,
)
from ..group_size_validation import validate_group_size_divisibility

__all__ = ["QuantizationMixin", "KV_CACHE_TARGETS"]

# attention modules are found by name, as in the reference (compressed-tensors KV_CACHE_TARGETS)
KV_CACHE_TARGETS = ["re:.*self_attn$"]


class _ObservedKVCache:
    """Stands in for the attention module's ``past_key_values`` during calibration: ``update`` shows the key
    and value states (keys after the rotary embedding, as they would enter the cache) to the module's
    observers, then defers to the real cache, or hands the states back when there is none."""

    def __init__(self, module, inner):
        self._module, self._inner = module, inner

    def update(self, key_states, value_states, *args, **kwargs):
        calibrate_key_hook(self._module, key_states)
        calibrate_value_hook(self._module, value_states)
        if self._inner is not None:
            return self._inner.update(key_states, value_states, *args, **kwargs)
        return key_states, value_states

    def __getattr__(self, name):
        return getattr(self._inner, name)


def _kv_cache_pre_hook(module, args, kwargs):
    for name in ("past_key_values", "past_key_value"):
        if name in kwargs:
            kwargs[name] = _ObservedKVCache(module, kwargs[name])
            return args, kwargs
    kwargs["past_key_values"] = _ObservedKVCache(module, None)
    return args, kwargs


class QuantizationMixin(HooksMixin):
    config_groups: dict[str, QuantizationScheme] | None = None
    targets: str | list[str] = Field(default_factory=lambda: ["Linear"])
    ignore: list[str] = Field(default_factory=list)
    scheme: str | dict[str, Any] | None = None
    kv_cache_scheme: QuantizationArgs | None = None
    weight_observer: str | None = None
    input_observer: str | None = None
    output_observer: str | None = None
    observer: dict[str, str] | None = None
    bypass_divisibility_checks: bool = False

    _calibration_hooks: set = PrivateAttr(default_factory=set)
    _resolved_config: QuantizationConfig | None = PrivateAttr(None)

    @field_validator("targets", mode="before")
    def validate_targets(cls, value):
        return [value] if isinstance(value, str) else value

    @field_validator("scheme", mode="before")
    def validate_scheme(cls, value):
        if isinstance(value, str):
            if not is_preset_scheme(value):
                raise ValueError("`scheme` must either be a preset scheme name or a dictionary of preset scheme names")
        elif isinstance(value, dict):
            for name in value.keys():
                cls.validate_scheme(name)
            for key, target in value.items():
                value[key] = cls.validate_targets(target)
        return value

    @field_validator("observer", mode="before")
    def validate_observer(cls, value):
        if value is None:
            return value
        if not isinstance(value, dict):
            raise ValueError("`observer` must be a dictionary")
        valid = {"weights", "input", "output"}
        for key in value.keys():
            if key not in valid:
                raise ValueError(f"Invalid observer key '{key}'. Valid keys are: {valid}")
            if not isinstance(value[key], str):
                raise ValueError(f"Observer value for '{key}' must be a string")
        return value

    @property
    def resolved_config(self) -> QuantizationConfig:
        if self._resolved_config is None:
            self._resolved_config = self.resolve_quantization_config()
        return self._resolved_config

    @property
    def resolved_targets(self) -> set[str]:
        targets = set()
        for group in self.resolved_config.config_groups.values():
            targets.update(group.targets)
        if self.resolved_config.kv_cache_scheme is not None:
            targets.update(KV_CACHE_TARGETS)
        return targets

    def initialize_quantization(self, model: torch.nn.Module):
        for _, module in match_named_modules(model, self.resolved_targets, self.ignore):
            reset_quantization_status(module)
        apply_quantization_config(model, self.resolved_config)
        self._initialize_kv_cache(model)
        if not self.bypass_divisibility_checks:
            validate_group_size_divisibility(model, self.resolved_targets, self.ignore)
        model.apply(disable_quantization)

    def start_calibration(self, model: torch.nn.Module):
        for _, module in match_named_modules(model, self.resolved_targets, self.ignore):
            self._initialize_observers(module)
            self._calibration_hooks |= self._initialize_hooks(module)
            apply_calibration_status(module)
        fuse_weight_observers(model)

    def end_calibration(self, model: torch.nn.Module):
        self.remove_hooks(self._calibration_hooks)
        self._calibration_hooks = set()
        for _, module in match_named_modules(model, self.resolved_targets, self.ignore):
            freeze_module_quantization(module)
        model.apply(enable_quantization)

    def sync_obs_act_stats(self, modules: Iterator[torch.nn.Module]):
        """Single-GPU build: activation statistics need no cross-rank reduction."""
        return

    @model_validator(mode="after")
    def _set_requires_calibration_data(self):
        if self.requires_calibration_data:
            return self
        if self.kv_cache_scheme is not None:
            self.requires_calibration_data = True
            return self
        for scheme in self.resolved_config.config_groups.values():
            if scheme.weights is not None and scheme.weights.observer == "imatrix_mse":
                self.requires_calibration_data = True
                return self
            if scheme.input_activations is not None and scheme.input_activations.dynamic in (False, DynamicType.LOCAL):
                self.requires_calibration_data = True
                return self
            if scheme.output_activations is not None and not scheme.output_activations.dynamic:
                self.requires_calibration_data = True
                return self
        return self

    def has_config(self) -> bool:
        return not (self.config_groups is None and self.targets == ["Linear"] and self.ignore == []
                    and self.scheme is None and self.kv_cache_scheme is None)

    def resolve_quantization_config(self) -> QuantizationConfig:
        scheme, targets, config_groups = self.scheme, self.targets, self.config_groups
        if scheme is not None and config_groups is not None:
            raise ValueError("Please specify either `scheme` or `config_groups`")
        if scheme is not None:
            if isinstance(scheme, str) and is_preset_scheme(scheme):
                scheme = {scheme: targets}
            config_groups = {}
            for idx, key in enumerate(scheme.keys()):
                if is_preset_scheme(key):
                    obj = preset_name_to_scheme(key, scheme[key])
                else:
                    obj = QuantizationScheme.model_validate({"targets": scheme[key], **scheme})
                config_groups[f"group_{idx}"] = self._apply_observer_overrides(obj)
        if config_groups is None or len(config_groups) == 0:
            config_groups = {"group_0": self._apply_observer_overrides(QuantizationScheme(targets=targets))}
        elif scheme is None:
            config_groups = {k: (v if isinstance(v, QuantizationScheme) else QuantizationScheme.model_validate(v))
                             for k, v in config_groups.items()}
            for obj in config_groups.values():
                self._apply_observer_overrides(obj)
        return QuantizationConfig(config_groups=config_groups, kv_cache_scheme=self.kv_cache_scheme,
                                  quantization_status=QuantizationStatus.INITIALIZED, ignore=self.ignore)

    def _apply_observer_overrides(self, scheme: QuantizationScheme) -> QuantizationScheme:
        individual = any(o is not None for o in (self.weight_observer, self.input_observer, self.output_observer))
        if individual and self.observer is not None:
            raise ValueError("Cannot specify both individual observer parameters (weight_observer, input_observer, "
                             "output_observer) and observer dict. Please use either individual parameters or the "
                             "observer dict.")
        w, i, o = self.weight_observer, self.input_observer, self.output_observer
        if self.observer is not None:
            w = self.observer.get("weights", w)
            i = self.observer.get("input", i)
            o = self.observer.get("output", o)
        for value, attr in ((w, "weights"), (i, "input_activations"), (o, "output_activations")):
            q_args = getattr(scheme, attr, None)
            if value is not None and q_args is not None:
                d = q_args.model_dump()
                d["observer"] = value
                setattr(scheme, attr, QuantizationArgs.model_validate(d))
        return scheme

    def _initialize_kv_cache(self, model: torch.nn.Module):
        """Attention modules get a scheme whose input arguments are the kv-cache arguments and ``k_scale`` /
        ``v_scale`` parameters (reference: mixin.py:216-218,342-383; compressed-tensors initialises the
        parameters from the observed shape (kv heads, head dim)).  Their forward is not wrapped: the scales are
        calibrated for the serving engine's cache, the calibration forward itself stays unquantised."""
        kv_args = self.resolved_config.kv_cache_scheme
        if kv_args is None:
            return
        from ....quantization.lifecycle import initialize_qparams

        for _, module in match_named_modules(model, KV_CACHE_TARGETS, self.ignore):
            config = getattr(module, "config", None)
            heads = getattr(config, "num_key_value_heads", None) or getattr(config, "num_attention_heads", None)
            head_dim = getattr(module, "head_dim", None)
            if heads is None or head_dim is None:
                raise ValueError("kv_cache_scheme: attention modules need `config.num_key_value_heads` and "
                                 f"`head_dim` (found {type(module).__name__})")
            module.quantization_scheme = QuantizationScheme(targets=list(KV_CACHE_TARGETS), input_activations=kv_args)
            module.quantization_status = QuantizationStatus.INITIALIZED
            module._llmc_kv_cache = True
            dtype = next(module.parameters()).dtype
            for base in ("k", "v"):
                initialize_qparams(module, base, kv_args, (heads, head_dim), dtype, force_zero_point=False)

    def _initialize_observers(self, module: torch.nn.Module):
        if not hasattr(module, "quantization_scheme"):
            return
        scheme: QuantizationScheme = module.quantization_scheme
        if getattr(module, "_llmc_kv_cache", False):
            if scheme.input_activations.dynamic in (False, DynamicType.LOCAL):
                initialize_observer(module, base_name="k")
                initialize_observer(module, base_name="v")
            return
        inp = scheme.input_activations and scheme.input_activations.dynamic in (False, DynamicType.LOCAL)
        out = scheme.output_activations and not scheme.output_activations.dynamic
        if inp:
            initialize_observer(module, base_name="input")
        if scheme.weights is not None:
            initialize_observer(module, base_name="weight")
        if out:
            initialize_observer(module, base_name="output")

    def _initialize_hooks(self, module: torch.nn.Module) -> set:
        hooks = set()
        if not hasattr(module, "quantization_scheme"):
            return hooks
        scheme: QuantizationScheme = module.quantization_scheme
        inp = scheme.input_activations and scheme.input_activations.dynamic in (False, DynamicType.LOCAL)
        out = scheme.output_activations and not scheme.output_activations.dynamic
        if getattr(module, "_llmc_kv_cache", False):
            if inp:
                hooks.add(self.register_hook(module, _kv_cache_pre_hook, "forward_pre", with_kwargs=True))
            return hooks
        if inp:
            hooks.add(self.register_hook(module, calibrate_input_hook, "forward_pre"))
        if out:
            hooks.add(self.register_hook(module, calibrate_output_hook, "forward"))
        return hooks
