"""Scheme registry and backend selection.

Same contract as the reference's registry (entropack/registry.py:24-121): schemes register by name; `select`
returns the lane name for a (scheme, tensor, requested backend) triple, trying backends by descending priority
and raising `DispatchError` with one reason per rejected backend, so that no fallback is ever silent.
"""
import logging
import threading

import torch

from .backends import BACKENDS, Backend

log = logging.getLogger("entropack.registry")

CONTAINER_DTYPES = (
    torch.float32, torch.float16, torch.bfloat16,
    torch.float8_e4m3fn, torch.float8_e4m3fnuz, torch.float8_e5m2, torch.float8_e5m2fnuz,
    torch.int64, torch.int32, torch.int16, torch.int8, torch.uint64, torch.uint32, torch.uint16, torch.uint8, torch.bool,
)

_guard = threading.Lock()
_scheme_table: dict[str, object] = {}
_backend_table: dict[str, Backend] = {spec.name: spec for spec in BACKENDS}
_probe_results: dict[str, str | None] = {}


class DispatchError(RuntimeError):
    """No backend could take the request. `reasons` maps each backend considered to why it was turned down."""

    def __init__(self, scheme: str, reasons: dict[str, str]):
        self.scheme = scheme
        self.reasons = dict(reasons)
        text = f"No backend can handle '{scheme}'"
        if self.reasons:
            text += ": " + "; ".join(f"{name}: {why}" for name, why in self.reasons.items())
        super().__init__(text)


def register_scheme(scheme):
    with _guard:
        _scheme_table[scheme.name] = scheme
    return scheme


def get_scheme(name: str):
    scheme = _scheme_table.get(name)
    if scheme is None:
        raise KeyError(f"Unknown scheme '{name}'; available: {sorted(_scheme_table)}")
    return scheme


def all_schemes() -> list:
    return sorted(_scheme_table.values(), key=lambda s: (-s.priority, s.name))


def name_for_config(config) -> str:
    for klass in type(config).__mro__:
        for scheme in _scheme_table.values():
            if scheme.config_cls is klass:
                return scheme.name
    raise TypeError(f"{type(config).__name__} is not the config of any registered scheme")


def require_dtype(dtype: torch.dtype) -> torch.dtype:
    if dtype not in CONTAINER_DTYPES:
        raise ValueError(f"Unsupported tensor dtype {dtype}; supported: {sorted(CONTAINER_DTYPES, key=str)}")
    return dtype


def default_config(dtype, **overrides):
    dtype = require_dtype(dtype)
    for scheme in all_schemes():
        if scheme.supports(dtype):
            return scheme.make_config({**scheme.options_for(dtype), **overrides})
    raise ValueError(f"no registered scheme supports {dtype}")


def reason(backend: str) -> str | None:
    """Why `backend` cannot be used (None = it can). Each probe runs once; its answer is kept."""
    spec = _backend_table.get(backend)
    if spec is None:
        return "not registered"
    if backend not in _probe_results:
        with _guard:
            if backend not in _probe_results:
                _probe_results[backend] = None if spec.probe is None else spec.probe()
    return _probe_results[backend]


def _turned_down(name: str, scheme, dtype) -> str | None:
    if name not in _backend_table:
        return "not registered"
    if name not in scheme.lanes:
        return f"scheme '{scheme.name}' declares no '{name}' lane"
    why = reason(name)
    if why is not None:
        return why
    if dtype is not None and not scheme.supports(dtype):
        return f"dtype {dtype} is not supported"
    return None


def select(scheme, tensor: torch.Tensor | None = None, backend: str | None = None, *, gate_dtype: bool = True) -> str:
    dtype = tensor.dtype if (gate_dtype and tensor is not None) else None
    if backend is not None:
        why = _turned_down(backend, scheme, dtype)
        if why is not None:
            raise DispatchError(scheme.name, {backend: why})
        log.debug("Backend %s selected for %s", backend, scheme.name)
        return backend
    turned_down: dict[str, str] = {}
    for spec in sorted(_backend_table.values(), key=lambda b: -b.priority):
        why = _turned_down(spec.name, scheme, dtype)
        if why is None:
            log.debug("Backend %s selected for %s", spec.name, scheme.name)
            return spec.name
        turned_down[spec.name] = why
    raise DispatchError(scheme.name, turned_down)


def backend_device(backend: str | None) -> torch.device | None:
    spec = _backend_table.get(backend) if backend is not None else None
    if spec is None or spec.device is None:
        return None
    return spec.device()
