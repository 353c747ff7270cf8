"""Execution backends a scheme lane can run on.

Mirrors the reference's backend table (entropack/backends/__init__.py:9-19): a backend is a name, a priority, a
`probe` returning None or the reason it is unusable, and the device its lanes run on. Here the accelerated
backend is `hip` (MI355X); `eager` is the CPU side, which in this package only encodes.
"""
from collections.abc import Callable
from dataclasses import dataclass

import torch

from . import hip


@dataclass(frozen=True)
class Backend:
    name: str
    priority: int = 0
    probe: Callable[[], str | None] | None = None
    device: Callable[[], torch.device] | None = None


BACKENDS: tuple[Backend, ...] = (
    Backend("hip", priority=200, probe=hip.probe, device=hip.runs_on),
    Backend("eager", priority=0),
)
