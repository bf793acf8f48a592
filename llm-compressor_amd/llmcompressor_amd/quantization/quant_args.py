"""Quantization argument / scheme / config types.

The reference takes these from compressed-tensors (``QuantizationArgs``,
``QuantizationScheme``, ``QuantizationConfig``, the preset scheme table; used at
``src/llmcompressor/modifiers/quantization/quantization/mixin.py:127-140,335-386``).
That package is not a dependency here, so the types are restated with the same
field names, defaults and validation so that recipes and modifier arguments
written for the reference load unchanged.
"""
from __future__ import annotations

from copy import deepcopy
from enum import Enum
from typing import Any, Dict, List, Optional, Union

import torch
from pydantic import BaseModel, ConfigDict, Field, field_serializer, field_validator, model_validator

__all__ = [
    "QuantizationType",
    "QuantizationStrategy",
    "ActivationOrdering",
    "DynamicType",
    "QuantizationStatus",
    "QuantizationArgs",
    "QuantizationScheme",
    "QuantizationConfig",
    "PRESET_SCHEMES",
    "is_preset_scheme",
    "preset_name_to_scheme",
    "FP8_E4M3_DATA",
    "FP4_E2M1_DATA",
]


class QuantizationType(str, Enum):
    INT = "int"
    FLOAT = "float"


class QuantizationStrategy(str, Enum):
    TENSOR = "tensor"
    CHANNEL = "channel"
    GROUP = "group"
    BLOCK = "block"
    TOKEN = "token"
    TENSOR_GROUP = "tensor_group"
    ATTN_HEAD = "attn_head"


class DynamicType(str, Enum):
    LOCAL = "local"


class ActivationOrdering(str, Enum):
    """group ("dynamic"): permute columns and emit g_idx; weight ("static"): permute only while quantising.

    "dynamic"/"static" are aliases: members compare (and hash) equal to their canonical name and to the
    plain strings, as the reference's enum does.
    """

    GROUP = "group"
    WEIGHT = "weight"
    DYNAMIC = "dynamic"
    STATIC = "static"

    @staticmethod
    def get_aliases():
        return {"dynamic": "group", "static": "weight"}

    @staticmethod
    def _canon(v):
        if isinstance(v, Enum):
            v = v.value
        if isinstance(v, str):
            v = v.lower()
            return ActivationOrdering.get_aliases().get(v, v)
        return v

    def __eq__(self, other):
        if other is None or isinstance(other, bool):
            return False
        return ActivationOrdering._canon(self) == ActivationOrdering._canon(other)

    def __ne__(self, other):
        return not self.__eq__(other)

    def __hash__(self):
        return hash(ActivationOrdering._canon(self))


class QuantizationStatus(str, Enum):
    INITIALIZED = "initialized"
    CALIBRATION = "calibration"
    FROZEN = "frozen"
    COMPRESSED = "compressed"


class _FloatData:
    def __init__(self, max_, dtype):
        self.max = max_
        self.min = -max_
        self.dtype = dtype


FP8_E4M3_DATA = _FloatData(448.0, torch.float8_e4m3fn)
FP4_E2M1_DATA = _FloatData(6.0, None)

_DTYPE_NAMES = {
    "float8_e4m3fn": torch.float8_e4m3fn,
    "uint8": torch.uint8,
    "int8": torch.int8,
    "int32": torch.int32,
    "bfloat16": torch.bfloat16,
    "float16": torch.float16,
    "float32": torch.float32,
}


def _parse_dtype(v):
    if v is None or isinstance(v, torch.dtype):
        return v
    name = str(v).replace("torch.", "")
    if name not in _DTYPE_NAMES:
        raise ValueError(f"unknown dtype {v}")
    return _DTYPE_NAMES[name]


class QuantizationArgs(BaseModel):
    model_config = ConfigDict(arbitrary_types_allowed=True, extra="forbid", use_enum_values=False)

    num_bits: int = 8
    type: QuantizationType = QuantizationType.INT
    symmetric: bool = True
    group_size: Optional[int] = None
    strategy: Optional[QuantizationStrategy] = None
    block_structure: Optional[List[int]] = None
    dynamic: Union[DynamicType, bool] = False
    actorder: Union[ActivationOrdering, bool, None] = None
    scale_dtype: Optional[Any] = None
    zp_dtype: Optional[Any] = None
    observer: Optional[str] = Field(default=None)
    observer_kwargs: Dict[str, Any] = Field(default_factory=dict)

    @field_validator("type", mode="before")
    def _v_type(cls, v):
        return v.lower() if isinstance(v, str) else v

    @field_validator("group_size", mode="before")
    def _v_group(cls, v):
        if v is None:
            return v
        if v < -1:
            raise ValueError(f"Invalid group size {v}. Use group_size > 0 for strategy='group' and "
                             "group_size = -1 for 'channel'")
        return v

    @field_validator("block_structure", mode="before")
    def _v_block(cls, v):
        if v is None:
            return v
        if isinstance(v, str):
            v = [int(x) for x in v.split("x")]
        if len(v) != 2 or any((not isinstance(x, int)) or x <= 0 for x in v):
            raise ValueError(f"Invalid block_structure '{v}'. Must be a list of two ints [rows, cols].")
        return list(v)

    @field_validator("strategy", mode="before")
    def _v_strategy(cls, v):
        return v.lower() if isinstance(v, str) else v

    @field_validator("actorder", mode="before")
    def _v_actorder(cls, v):
        if isinstance(v, bool):
            return ActivationOrdering.GROUP if v else None
        if isinstance(v, str):
            return ActivationOrdering(v.lower())
        return v

    @field_validator("dynamic", mode="before")
    def _v_dynamic(cls, v):
        if isinstance(v, str):
            return DynamicType(v.lower())
        return v

    @field_validator("scale_dtype", "zp_dtype", mode="before")
    def _v_dtype(cls, v):
        return _parse_dtype(v)

    @field_serializer("scale_dtype", "zp_dtype")
    def _s_dtype(self, v):
        return None if v is None else str(v).replace("torch.", "")

    @field_serializer("type", "strategy", "actorder", "dynamic")
    def _s_enum(self, v):
        return v.value if isinstance(v, Enum) else v

    @model_validator(mode="after")
    def _validate(self):
        strategy, group_size, actorder, dynamic = self.strategy, self.group_size, self.actorder, self.dynamic
        if strategy is None:
            if self.block_structure is not None:
                strategy = QuantizationStrategy.BLOCK
            elif group_size is None:
                strategy = QuantizationStrategy.TENSOR
            elif group_size > 0:
                strategy = QuantizationStrategy.GROUP
            elif group_size == -1:
                strategy = QuantizationStrategy.CHANNEL
            else:
                raise ValueError(f"Invalid group size {group_size}")
        if strategy in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP):
            if group_size is None or group_size <= 0:
                raise ValueError(f"strategy {strategy.value} requires group_size to be set to a positive value")
        elif group_size is not None and group_size > 0:
            raise ValueError("group_size requires strategy to be set to 'group' or 'tensor_group'")
        if strategy == QuantizationStrategy.BLOCK and self.block_structure is None:
            raise ValueError("strategy 'block' requires block_structure")
        if dynamic is True:
            if strategy not in (QuantizationStrategy.TOKEN, QuantizationStrategy.TENSOR,
                                QuantizationStrategy.TENSOR_GROUP, QuantizationStrategy.GROUP):
                raise ValueError("dynamic quantization is only supported for token, tensor, group and tensor_group")
            if self.observer is not None:
                if self.observer != "memoryless":
                    self.observer = None
        elif self.observer is None:
            self.observer = "minmax"
        if self.zp_dtype is None:
            self.zp_dtype = self.pytorch_dtype()
        self.strategy = strategy
        return self

    def pytorch_dtype(self) -> torch.dtype:
        if self.type == QuantizationType.FLOAT:
            if self.num_bits == 8:
                return torch.float8_e4m3fn
            # fp4 codes have no torch storage type of their own; zero points are kept in e4m3
            return torch.float8_e4m3fn
        if self.num_bits <= 8:
            return torch.int8
        if self.num_bits <= 16:
            return torch.int16
        return torch.int32

    # helpers used by the kernel-facing code
    @property
    def is_fp4(self) -> bool:
        return self.type == QuantizationType.FLOAT and self.num_bits == 4

    @property
    def is_mx(self) -> bool:
        return self.is_fp4 and self.scale_dtype == torch.uint8

    def get_observer(self) -> Optional[str]:
        return self.observer


class QuantizationScheme(BaseModel):
    model_config = ConfigDict(extra="forbid")

    targets: List[str]
    weights: Optional[QuantizationArgs] = None
    input_activations: Optional[QuantizationArgs] = None
    output_activations: Optional[QuantizationArgs] = None
    format: Optional[str] = None

    @model_validator(mode="after")
    def _validate(self):
        for name in ("input_activations", "output_activations"):
            a = getattr(self, name)
            if a is not None and a.actorder is not None:
                raise ValueError("Cannot apply actorder to activations")
        return self


class QuantizationConfig(BaseModel):
    model_config = ConfigDict(extra="forbid")

    config_groups: Dict[str, Union[QuantizationScheme, List[str]]]
    quant_method: str = "compressed-tensors"
    kv_cache_scheme: Optional[QuantizationArgs] = None
    format: str = "dense"
    quantization_status: QuantizationStatus = QuantizationStatus.INITIALIZED
    global_compression_ratio: Optional[float] = None
    ignore: Optional[List[str]] = Field(default_factory=list)
    version: str = "llmcompressor_amd"

    @field_serializer("quantization_status")
    def _s_status(self, v):
        return v.value if isinstance(v, Enum) else v


def _w(**kw):
    return QuantizationArgs(**kw)


# preset table: same names and meanings as compressed-tensors' PRESET_SCHEMES
_PRESETS = {
    "UNQUANTIZED": dict(),
    "W8A16": dict(weights=dict(num_bits=8, type="int", symmetric=True, strategy="channel", dynamic=False)),
    "W4A16": dict(weights=dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128,
                               dynamic=False)),
    "W4A16_ASYM": dict(weights=dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128,
                                    dynamic=False)),
    "W8A8": dict(
        weights=dict(num_bits=8, type="int", symmetric=True, strategy="channel", dynamic=False),
        input_activations=dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True,
                               observer=None),
    ),
    "W4A8": dict(
        weights=dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128, dynamic=False),
        input_activations=dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True,
                               observer=None),
    ),
    # int4 group weights, fp8 per-token activations (reference: examples/quantization_w4a8_fp8/llama3_example.py:53)
    "W4AFP8": dict(
        weights=dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128, dynamic=False),
        input_activations=dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True,
                               observer=None),
    ),
    "FP8": dict(
        weights=dict(num_bits=8, type="float", symmetric=True, strategy="tensor", dynamic=False),
        input_activations=dict(num_bits=8, type="float", symmetric=True, strategy="tensor", dynamic=False),
    ),
    "FP8_DYNAMIC": dict(
        weights=dict(num_bits=8, type="float", symmetric=True, strategy="channel", dynamic=False),
        input_activations=dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True,
                               observer=None),
    ),
    "FP8_BLOCK": dict(
        weights=dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[128, 128],
                     dynamic=False),
        input_activations=dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128,
                               dynamic=True, observer=None),
    ),
    "NVFP4A16": dict(weights=dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group",
                                  group_size=16, dynamic=False, scale_dtype="float8_e4m3fn",
                                  zp_dtype="float8_e4m3fn")),
    "NVFP4": dict(
        weights=dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16,
                     dynamic=False, scale_dtype="float8_e4m3fn", zp_dtype="float8_e4m3fn"),
        input_activations=dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16,
                               dynamic="local", observer="static_minmax", scale_dtype="float8_e4m3fn",
                               zp_dtype="float8_e4m3fn"),
    ),
    "MXFP4A16": dict(weights=dict(num_bits=4, type="float", symmetric=True, strategy="group", group_size=32,
                                  dynamic=False, scale_dtype="uint8", zp_dtype="uint8")),
    "MXFP4": dict(
        weights=dict(num_bits=4, type="float", symmetric=True, strategy="group", group_size=32, dynamic=False,
                     scale_dtype="uint8", zp_dtype="uint8"),
        input_activations=dict(num_bits=4, type="float", symmetric=True, strategy="group", group_size=32,
                               dynamic=True, observer=None, scale_dtype="uint8", zp_dtype="uint8"),
    ),
}
_PRESETS["INT8"] = _PRESETS["W8A8"]
_PRESETS["FLOAT8"] = _PRESETS["FP8"]
PRESET_SCHEMES = _PRESETS


def is_preset_scheme(name: str) -> bool:
    return isinstance(name, str) and name.upper() in PRESET_SCHEMES


def preset_name_to_scheme(name: str, targets: List[str]) -> QuantizationScheme:
    name = name.upper()
    if name not in PRESET_SCHEMES:
        raise KeyError(f"Unknown preset scheme name {name}, available names: {list(PRESET_SCHEMES.keys())}")
    spec = deepcopy(PRESET_SCHEMES[name])
    return QuantizationScheme(targets=list(targets), **{k: QuantizationArgs(**v) for k, v in spec.items()})
