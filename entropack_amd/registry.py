"""Scheme registry and backend selection.

Module-level functions with the reference's names and meaning (entropack/registry.py:24-121) over one `_Registry`
object: schemes register by name; `select` answers which lane (= backend name) serves a (scheme, tensor, requested
backend) request, trying backends from the highest priority down, and raises `DispatchError` listing why each backend
was turned down, so no fallback is ever silent. A backend's probe runs once per process.
"""
import logging
import threading
from typing import Optional

import torch

from .backends import BACKENDS

log = logging.getLogger("entropack.registry")

CONTAINER_DTYPES = frozenset(
    [torch.bool, torch.bfloat16, torch.float16, torch.float32]
    + [torch.float8_e4m3fn, torch.float8_e4m3fnuz, torch.float8_e5m2, torch.float8_e5m2fnuz]
    + [torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8, torch.uint16, torch.uint32, torch.uint64]
)


class DispatchError(RuntimeError):
    """No backend could take the request. `reasons` maps each backend considered to why it was turned down."""

    def __init__(self, scheme: str, reasons: dict):
        self.scheme, self.reasons = scheme, dict(reasons)
        listed = "; ".join(f"{backend}: {why}" for backend, why in self.reasons.items())
        super().__init__(f"No backend can handle '{scheme}'" + (": " + listed if listed else ""))


class _Registry:
    def __init__(self, backends):
        self.lock = threading.Lock()
        self.schemes = {}
        self.backends = {record.name: record for record in backends}
        self.by_priority = sorted(self.backends.values(), key=lambda record: record.priority, reverse=True)
        self.probed = {}                                       # backend name -> None (usable) or the reason it is not

    def add(self, scheme):
        with self.lock:
            self.schemes[scheme.name] = scheme
        return scheme

    def ranked_schemes(self) -> list:
        return sorted(self.schemes.values(), key=lambda scheme: (-scheme.priority, scheme.name))

    def availability(self, backend: str) -> Optional[str]:
        record = self.backends.get(backend)
        if record is None:
            return "not registered"
        with self.lock:
            if backend not in self.probed:
                self.probed[backend] = record.probe() if record.probe else None
            return self.probed[backend]

    def objection(self, backend: str, scheme, dtype) -> Optional[str]:
        """Why `backend` cannot serve `scheme` for `dtype` (None = it can)."""
        if backend not in self.backends:
            return "not registered"
        if backend not in scheme.lanes:
            return f"scheme '{scheme.name}' declares no '{backend}' lane"
        unavailable = self.availability(backend)
        if unavailable is not None:
            return unavailable
        if dtype is not None and not scheme.supports(dtype):
            return f"dtype {dtype} is not supported"
        return None

    def choose(self, scheme, dtype, requested: Optional[str]) -> str:
        candidates = [requested] if requested is not None else [record.name for record in self.by_priority]
        objections = {}
        for backend in candidates:
            why = self.objection(backend, scheme, dtype)
            if why is None:
                log.debug("Backend %s selected for %s", backend, scheme.name)
                return backend
            objections[backend] = why
        raise DispatchError(scheme.name, objections)


_registry = _Registry(BACKENDS)


def register_scheme(scheme):
    return _registry.add(scheme)


def get_scheme(name: str):
    if name not in _registry.schemes:
        raise KeyError(f"Unknown scheme '{name}'; available: {sorted(_registry.schemes)}")
    return _registry.schemes[name]


def all_schemes() -> list:
    return _registry.ranked_schemes()


def name_for_config(config) -> str:
    """The scheme whose config class `config` is an instance of (nearest class first)."""
    owners = {scheme.config_cls: scheme.name for scheme in _registry.schemes.values()}
    for klass in type(config).__mro__:
        if klass in owners:
            return owners[klass]
    raise TypeError(f"{type(config).__name__} is not the config of any registered scheme")


def require_dtype(dtype: torch.dtype) -> torch.dtype:
    if dtype not in CONTAINER_DTYPES:
        raise ValueError(f"Unsupported tensor dtype {dtype}; supported: {sorted(map(str, CONTAINER_DTYPES))}")
    return dtype


def default_config(dtype, **overrides):
    """The config of the highest-priority scheme that stores `dtype`, with that scheme's options for it."""
    require_dtype(dtype)
    for scheme in _registry.ranked_schemes():
        if scheme.supports(dtype):
            options = dict(scheme.options_for(dtype))
            options.update(overrides)
            return scheme.make_config(options)
    raise ValueError(f"no registered scheme supports {dtype}")


def reason(backend: str) -> Optional[str]:
    """Why `backend` cannot be used (None = it can)."""
    return _registry.availability(backend)


def select(scheme, tensor: Optional[torch.Tensor] = None, backend: Optional[str] = None, *, gate_dtype: bool = True) -> str:
    dtype = tensor.dtype if gate_dtype and tensor is not None else None
    return _registry.choose(scheme, dtype, backend)


def backend_device(backend: Optional[str]) -> Optional[torch.device]:
    record = _registry.backends.get(backend)
    return record.device() if record is not None and record.device is not None else None
