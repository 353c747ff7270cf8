"""Scheme base class: a named codec whose work is done by per-backend lane modules.

Public contract = the reference's (entropack/schemes/base.py:40-98), so that scheme packages and lanes written against
either code base plug into the other: class attributes `name`, `buffer_names`, `lossless`, `priority`, `dtypes`,
`lanes` (backend name -> module name inside the scheme's package); `lane(backend)` imports that module on first use;
`lane_for(tensor, backend)` lets the registry pick the backend; lane modules expose module-level `encode(...)` /
`decode(...)`; a scheme's config class is whatever its `encode` annotates `config` with.
"""
import dataclasses
import importlib
import typing
from abc import ABC, abstractmethod

import torch

from ..registry import DispatchError, backend_device, register_scheme, select
from .config import CompressionConfig, RawConfig, validate_config

__all__ = ["RawScheme", "Scheme", "cached_parse", "host_copy", "packed_buffers", "register_scheme"]


def packed_buffers(packed: dict, kind: type):
    """A scheme's buffers, picked out of a name -> tensor mapping in the order of its NamedTuple `kind`."""
    return kind._make(packed[field] for field in kind._fields)


#: Attribute a device-resident buffer view carries when a host copy of the same values came along with it (containers
#: attach it when they move to a device), and the largest buffer that gets one.
HOST_MIRROR = "_entropack_host_mirror"
HOST_MIRROR_LIMIT = 64 * 1024


def host_copy(tensor: torch.Tensor) -> torch.Tensor:
    """The values of a small metadata buffer on the host: the copy that travelled with it, else a read-back."""
    mirror = getattr(tensor, HOST_MIRROR, None)
    return mirror if mirror is not None else tensor.detach().cpu()


def cached_parse(tensor: torch.Tensor, parse, attribute: str):
    """`parse(tensor)`, computed once per tensor object and kept on it (small metadata tensors: layouts, lane modes)."""
    try:
        return getattr(tensor, attribute)
    except AttributeError:
        value = parse(tensor)
        setattr(tensor, attribute, value)
        return value


class _LaneModules:
    """Lane modules by (scheme class, backend), imported when first asked for."""

    def __init__(self):
        self._loaded = {}

    def get(self, scheme: "Scheme", backend: str):
        owner = type(scheme)
        try:
            return self._loaded[owner, backend]
        except KeyError:
            pass
        module_name = scheme.lanes.get(backend)
        if module_name is None:
            raise DispatchError(scheme.name, {backend: f"scheme '{scheme.name}' declares no '{backend}' lane"})
        try:
            module = importlib.import_module("." + module_name, package=owner.__module__)
        except Exception as error:
            raise DispatchError(scheme.name, {backend: f"lane module failed to import: {error!r}"}) from error
        self._loaded[owner, backend] = module
        return module


_lane_modules = _LaneModules()
_config_classes: dict = {}


class Scheme(ABC):
    #: registry key and `compress_method` of the containers this scheme writes
    name: str
    #: names of the tensors a container of this scheme holds, in blob order
    buffer_names: tuple
    lossless: bool = True
    #: the scheme with the highest priority that supports a dtype is that dtype's default
    priority: int = 0
    #: dtypes the scheme encodes; None = any
    dtypes: typing.Optional[tuple] = None
    #: backend name -> lane module name, relative to the scheme's package
    lanes: dict = {}

    # -- what a scheme implements -----------------------------------------------------------------------------------

    @abstractmethod
    def encode(self, weight, config: CompressionConfig) -> dict:
        """tensor -> {buffer name: tensor}"""

    @abstractmethod
    def decode(self, packed: dict, *, shape, dtype, config: CompressionConfig):
        """{buffer name: tensor} -> tensor of `shape` and `dtype`"""

    def validate_buffers(self, buffers: dict, shape, dtype) -> None:
        """Raise ValueError / TypeError if `buffers` cannot be a container of `shape` and `dtype`."""

    def options_for(self, dtype: torch.dtype) -> dict:
        """Config options a layer uses for `dtype` when it was given no config."""
        return {}

    # -- what it inherits ---------------------------------------------------------------------------------------------

    def supports(self, dtype: torch.dtype) -> bool:
        return True if self.dtypes is None else dtype in self.dtypes

    def lane(self, backend: str):
        return _lane_modules.get(self, backend)

    def lane_for(self, tensor: typing.Optional[torch.Tensor] = None, backend: typing.Optional[str] = None, *, gate_dtype: bool = True):
        """(lane module, device its work runs on) for `tensor`; `backend` None or "auto" lets the registry choose."""
        wanted = backend if backend not in (None, "auto") else None
        chosen = select(self, tensor, wanted, gate_dtype=gate_dtype)
        return self.lane(chosen), backend_device(chosen)

    @property
    def config_cls(self) -> type:
        owner = type(self)
        if owner not in _config_classes:
            _config_classes[owner] = typing.get_type_hints(owner.encode)["config"]
        return _config_classes[owner]

    def make_config(self, options: dict):
        """This scheme's config from option names and values; unknown names and bad values both raise."""
        accepted = [field.name for field in dataclasses.fields(self.config_cls)]
        strangers = sorted(name for name in options if name not in accepted)
        if strangers:
            raise TypeError(f"Unknown {self.name} options: {strangers}")
        config = self.config_cls(**options)
        validate_config(config)
        return config


class RawScheme(Scheme):
    """Stores the tensor as is; what `compress` falls back to when a scheme cannot encode an input."""

    name = "raw"
    buffer_names = ("data",)
    priority = -1

    def encode(self, weight, config: RawConfig) -> dict:
        return {"data": weight.detach().contiguous().clone()}

    def decode(self, packed: dict, *, shape, dtype, config: RawConfig) -> torch.Tensor:
        return packed["data"]

    def validate_buffers(self, buffers, shape, dtype) -> None:
        data = buffers["data"]
        if (data.dtype, tuple(data.shape)) != (dtype, tuple(shape)):
            raise ValueError(f"raw buffer must be {tuple(shape)} {dtype}, got {tuple(data.shape)} {data.dtype}")


register_scheme(RawScheme())
