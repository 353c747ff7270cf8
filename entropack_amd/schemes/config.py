"""Config dataclasses and their validation.

Same user-facing contract as the reference (entropack/schemes/config.py:8-111): every scheme has a dataclass
deriving from `CompressionConfig`; fields carry `Annotated[type, Range | OneOf]` markers; `validate_config` raises
TypeError for a wrong kind of value and ValueError for one outside its marker. `execution_backend` is not
validated here: any string reaches the registry, which rejects unknown names with a DispatchError.
"""
from dataclasses import dataclass, fields
from numbers import Real
from typing import Annotated, get_args, get_origin, get_type_hints

__all__ = ["CompressionConfig", "OneOf", "Range", "RawConfig", "validate_config"]


@dataclass
class CompressionConfig:
    """Execution settings shared by all schemes. Pick a concrete subclass to pick a scheme."""

    #: "auto" / None picks the best usable backend; otherwise "hip" or "eager".
    execution_backend: str | None = "auto"


@dataclass
class RawConfig(CompressionConfig):
    """Keep the values as they are (no entropy coding)."""


class Range:
    """Inclusive bounds; None leaves a side open."""

    def __init__(self, low=None, high=None, *, message: str | None = None):
        self.low, self.high, self.message = low, high, message

    def holds(self, value) -> bool:
        return (self.low is None or value >= self.low) and (self.high is None or value <= self.high)

    def describe(self, name: str) -> str:
        if self.message:
            return self.message
        if self.low is None:
            return f"{name} must be <= {self.high}"
        if self.high is None:
            return f"{name} must be >= {self.low}"
        return f"{name} must be in [{self.low}, {self.high}]"


class OneOf:
    """A closed set; `silent` values mean "choose for me" and pass as well."""

    def __init__(self, choices, *, silent=(), message: str | None = None):
        self.choices, self.silent, self.message = tuple(choices), frozenset(silent), message

    def holds(self, value) -> bool:
        return value in self.choices or value in self.silent

    def describe(self, name: str) -> str:
        return self.message or f"{name} must be one of {self.choices}"


_field_hints: dict[type, dict] = {}


def _hints_of(klass: type) -> dict:
    if klass not in _field_hints:
        hints = get_type_hints(klass, include_extras=True)
        _field_hints[klass] = {f.name: hints[f.name] for f in fields(klass) if f.name != "execution_backend"}
    return _field_hints[klass]


def _validate_field(name: str, value, hint) -> None:
    markers = ()
    if get_origin(hint) is Annotated:
        hint, *markers = get_args(hint)
    members = get_args(hint) if get_origin(hint) is not None else (hint,)
    kinds = [m for m in members if m is not type(None)]
    nullable = len(kinds) != len(members)
    base = kinds[0]
    noun = {int: "an integer", bool: "a bool"}.get(base, "a real number")
    if value is None:
        if nullable:
            return
        raise TypeError(f"{name} must be {noun}")
    if base is bool:
        right_kind = isinstance(value, bool)
    elif base is int:
        right_kind = isinstance(value, int) and not isinstance(value, bool)
    else:
        right_kind = isinstance(value, Real) and not isinstance(value, bool)
    if not right_kind:
        raise TypeError(f"{name} must be {noun}{' or None' if nullable else ''}")
    for marker in markers:
        if not marker.holds(value):
            raise ValueError(marker.describe(name))


def validate_config(config) -> None:
    for name, hint in _hints_of(type(config)).items():
        _validate_field(name, getattr(config, name), hint)
