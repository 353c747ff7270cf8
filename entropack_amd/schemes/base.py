"""Scheme base class: a named codec with per-backend lanes.

The contract follows the reference (entropack/schemes/base.py:40-98): a scheme lists `lanes` (backend name ->
module name inside the scheme's package); `lane_for` asks the registry which backend to use and imports that lane
module lazily; a lane module exposes module-level `encode(...)` / `decode(...)`. The config class of a scheme is
whatever its `encode` annotates `config` with.
"""
import importlib
from abc import ABC, abstractmethod
from dataclasses import fields
from typing import Any, get_type_hints

import torch

from ..registry import DispatchError, backend_device, register_scheme, select
from .config import CompressionConfig, RawConfig, validate_config

__all__ = ["RawScheme", "Scheme", "cached_parse", "packed_buffers", "register_scheme"]

_lanes_loaded: dict[tuple[type, str], Any] = {}
_config_of: dict[type, type] = {}


def packed_buffers(packed: dict, kind: type):
    """Pick a scheme's buffers out of a name -> tensor mapping, as its NamedTuple."""
    return kind(*(packed[name] for name in kind._fields))


def cached_parse(tensor: torch.Tensor, parse, attribute: str):
    """Parse a small metadata tensor once and keep the answer on the tensor object itself."""
    if not hasattr(tensor, attribute):
        setattr(tensor, attribute, parse(tensor))
    return getattr(tensor, attribute)


class Scheme(ABC):
    name: str
    buffer_names: tuple[str, ...]
    lossless: bool = True
    priority: int = 0
    dtypes: tuple[torch.dtype, ...] | None = None
    lanes: dict[str, str] = {}

    def supports(self, dtype: torch.dtype) -> bool:
        return self.dtypes is None or dtype in self.dtypes

    def options_for(self, dtype: torch.dtype) -> dict[str, Any]:
        return {}

    def lane(self, backend: str):
        key = (type(self), backend)
        if key not in _lanes_loaded:
            if backend not in self.lanes:
                raise DispatchError(self.name, {backend: f"scheme '{self.name}' declares no '{backend}' lane"})
            try:
                _lanes_loaded[key] = importlib.import_module("." + self.lanes[backend], package=type(self).__module__)
            except Exception as error:
                raise DispatchError(self.name, {backend: f"lane module failed to import: {error!r}"}) from error
        return _lanes_loaded[key]

    def lane_for(self, tensor: torch.Tensor | None = None, backend: str | None = None, *, gate_dtype: bool = True):
        chosen = select(self, tensor, None if backend in (None, "auto") else backend, gate_dtype=gate_dtype)
        return self.lane(chosen), backend_device(chosen)

    @abstractmethod
    def encode(self, weight, config: CompressionConfig) -> dict:
        ...

    @abstractmethod
    def decode(self, packed: dict, *, shape, dtype, config: CompressionConfig):
        ...

    @property
    def config_cls(self) -> type:
        klass = type(self)
        if klass not in _config_of:
            _config_of[klass] = get_type_hints(klass.encode)["config"]
        return _config_of[klass]

    def make_config(self, options: dict):
        known = {f.name for f in fields(self.config_cls)}
        unknown = sorted(set(options) - known)
        if unknown:
            raise TypeError(f"Unknown {self.name} options: {unknown}")
        config = self.config_cls(**options)
        validate_config(config)
        return config

    def validate_buffers(self, buffers: dict, shape, dtype) -> None:
        ...


class RawScheme(Scheme):
    """Stores the tensor as is; what `compress` falls back to when a scheme cannot encode an input."""

    name = "raw"
    buffer_names = ("data",)
    priority = -1
    dtypes = None
    lanes = {}

    def encode(self, weight, config: RawConfig) -> dict:
        return {"data": weight.detach().contiguous().clone()}

    def decode(self, packed: dict, *, shape, dtype, config: RawConfig) -> torch.Tensor:
        return packed["data"]

    def validate_buffers(self, buffers, shape, dtype) -> None:
        data = buffers["data"]
        if data.dtype != dtype or tuple(data.shape) != tuple(shape):
            raise ValueError(f"raw buffer must be {tuple(shape)} {dtype}, got {tuple(data.shape)} {data.dtype}")


register_scheme(RawScheme())
