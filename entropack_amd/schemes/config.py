"""Config dataclasses and their validation.

User-facing contract of the reference (entropack/schemes/config.py:8-111): every scheme has a dataclass deriving
from `CompressionConfig`; a field's annotation may carry constraint markers, `Annotated[int | None, Range(1, None)]`
or `Annotated[int, OneOf((9, 10), silent=(0,))]`; `validate_config` raises TypeError for the wrong kind of value and
ValueError for a value its markers refuse. `execution_backend` is left to the registry, which rejects unknown names
with a DispatchError.

Here a config class is compiled once into a list of `_Rule`s (kind of value, whether None passes, markers), and
validation walks that list.
"""
import dataclasses
import numbers
import typing
import weakref

__all__ = ["CompressionConfig", "OneOf", "Range", "RawConfig", "validate_config"]


@dataclasses.dataclass
class CompressionConfig:
    """Execution settings shared by all schemes. Pick a concrete subclass to pick a scheme."""

    #: "auto" / None picks the best usable backend; otherwise "hip" or "eager".
    execution_backend: typing.Optional[str] = "auto"


@dataclasses.dataclass
class RawConfig(CompressionConfig):
    """Keep the values as they are (no entropy coding)."""


class Range:
    """Marker: low <= value <= high, either side open when None. `message` replaces the generated complaint."""

    def __init__(self, low=None, high=None, *, message=None):
        self.low, self.high, self.message = low, high, message

    def refusal(self, name: str, value):
        """None if `value` passes, else the text of the ValueError."""
        below = self.low is not None and value < self.low
        above = self.high is not None and value > self.high
        if not (below or above):
            return None
        if self.message:
            return self.message
        if self.low is not None and self.high is not None:
            return f"{name} must be in [{self.low}, {self.high}]"
        return f"{name} must be >= {self.low}" if self.high is None else f"{name} must be <= {self.high}"


class OneOf:
    """Marker: value in a closed set; `silent` values mean "choose for me" and pass without being advertised."""

    def __init__(self, choices, *, silent=(), message=None):
        self.choices, self.silent, self.message = tuple(choices), tuple(silent), message

    def refusal(self, name: str, value):
        if value in self.choices or value in self.silent:
            return None
        return self.message or f"{name} must be one of {self.choices}"


class _Rule(typing.NamedTuple):
    name: str
    kind: type                  # bool, int or float ("any real number")
    none_passes: bool
    markers: tuple

    _NOUNS = {bool: "a bool", int: "an integer", float: "a real number"}

    def apply(self, value) -> None:
        noun = self._NOUNS[self.kind]
        if value is None:
            if not self.none_passes:
                raise TypeError(f"{self.name} must be {noun}")
            return
        is_bool = isinstance(value, bool)
        if self.kind is bool:
            fits = is_bool
        elif self.kind is int:
            fits = isinstance(value, int) and not is_bool
        else:
            fits = isinstance(value, numbers.Real) and not is_bool
        if not fits:
            raise TypeError(f"{self.name} must be {noun}" + (" or None" if self.none_passes else ""))
        for marker in self.markers:
            complaint = marker.refusal(self.name, value)
            if complaint is not None:
                raise ValueError(complaint)


def _rule_for(name: str, annotation) -> _Rule:
    markers = ()
    if typing.get_origin(annotation) is typing.Annotated:
        annotation, *found = typing.get_args(annotation)
        markers = tuple(found)
    alternatives = typing.get_args(annotation) or (annotation,)           # `int | None` -> (int, NoneType)
    concrete = [kind for kind in alternatives if kind is not type(None)]
    kind = concrete[0] if concrete[0] in (bool, int) else float
    return _Rule(name, kind, len(concrete) < len(alternatives), markers)


_compiled: dict = {}


def _rules(config_class: type) -> tuple:
    if config_class not in _compiled:
        annotations = typing.get_type_hints(config_class, include_extras=True)
        _compiled[config_class] = tuple(_rule_for(field.name, annotations[field.name]) for field in dataclasses.fields(config_class)
                                        if field.name != "execution_backend")
    return _compiled[config_class]


_last_valid: tuple = (None, None)      # (a weak reference to the config object validated last, the field values it had then)


def validate_config(config) -> None:
    # A layer validates the same config object on every forward: skip the rules while its fields are unchanged. The pair
    # is one tuple, read and replaced in one step, so two threads validating different configs can never pair one config's
    # identity with the other's fields; the config itself is held weakly.
    global _last_valid
    fields = getattr(config, "__dict__", None)
    seen, seen_fields = _last_valid
    if fields is not None and seen is not None and seen() is config and seen_fields == fields:
        return
    for rule in _rules(type(config)):
        rule.apply(getattr(config, rule.name))
    if fields is not None:
        try:
            _last_valid = (weakref.ref(config), dict(fields))
        except TypeError:          # a config type without weak references: validated every time
            pass
