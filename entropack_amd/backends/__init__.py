"""Execution backends a scheme lane can run on.

The registry asks four things of a backend record (same attribute names as the reference's table,
entropack/backends/__init__.py:9-19, so lanes written for either package resolve the same way): `name`, `priority`
(higher wins under "auto"), `probe()` -> None when usable or the reason why not, and `device()` -> where its lanes
run. `hip` is the MI355X backend; `eager` is the CPU side, which in this package only encodes.
"""
from typing import Callable, NamedTuple, Optional

import torch

from . import hip


class Backend(NamedTuple):
    name: str
    priority: int = 0
    probe: Optional[Callable[[], Optional[str]]] = None
    device: Optional[Callable[[], torch.device]] = None

    def unusable_because(self) -> Optional[str]:
        """None when lanes of this backend can run here, else a sentence for DispatchError."""
        return None if self.probe is None else self.probe()


def _table() -> tuple:
    accelerated = Backend(name="hip", priority=200, probe=hip.probe, device=hip.runs_on)
    host = Backend(name="eager")
    return tuple(sorted((accelerated, host), key=lambda record: -record.priority))


BACKENDS: tuple = _table()
