"""Unique default markers that survive copying and serialisation (reference: sentinel.py)."""
from __future__ import annotations

_registry: dict = {}


class Sentinel:
    def __new__(cls, name: str):
        if name not in _registry:
            obj = super().__new__(cls)
            obj.name = name
            _registry[name] = obj
        return _registry[name]

    def __repr__(self):
        return f"Sentinel({self.name!r})"

    def __eq__(self, other):
        return isinstance(other, Sentinel) and other.name == self.name

    def __hash__(self):
        return hash(("Sentinel", self.name))

    def __deepcopy__(self, memo):
        return self

    def __reduce__(self):
        return (Sentinel, (self.name,))

    @classmethod
    def __get_pydantic_core_schema__(cls, _source, _handler):
        from pydantic_core import core_schema

        def validate(v):
            if isinstance(v, Sentinel):
                return v
            if isinstance(v, str) and v.startswith("Sentinel("):
                return Sentinel(v[len("Sentinel('"):-2])
            raise ValueError("not a sentinel")

        return core_schema.no_info_plain_validator_function(
            validate, serialization=core_schema.plain_serializer_function_ser_schema(lambda v: v.name))
