"""`hip` lane of lattice_rans: decode on an MI355X through the C ABI of libentropack_hip.so.

Module-level `decode(buffers, *, shape, dtype, threads_per_block, l2_prefetch)` is the lane contract of the
reference's CUDA lane (entropack/schemes/lattice_rans/cuda.py:781-805): all buffers on the device, result
`[rows, padded cols]` of `dtype` on the same device, enqueued on torch's current stream without a host
synchronisation after the launch. Derived decode tables live in a plan cached on the `layout` tensor object and keyed
by the data pointers it was built from (cuda.py:697-741); the tables themselves are built by a device kernel.

There is no CPU path in this module and no fallback: a missing library or device raises.
"""
import ctypes
from dataclasses import dataclass

import numpy as np
import torch

from ...backends import hip as _hip
from .format import LatticeBuffers, decode_geometry, snap_to_container

#: float8 formats without a store kernel are decoded to float32 and cast on the device, as the reference does.
_VIA_FLOAT32 = frozenset({torch.float8_e4m3fnuz, torch.float8_e5m2fnuz})

#: Test hook: force one ep_hip_table_kind for every new plan (None = let the library choose).
FORCE_TABLE_KIND: int | None = None


@dataclass
class DecodePlan:
    desc: _hip.PlanDesc
    tables: torch.Tensor          # uint8, device; header + slot tables
    error: torch.Tensor           # int32[1], device; first decode error of any launch using this plan
    key: tuple

    @property
    def table_kind(self) -> str:
        return _hip.TABLE_KIND_NAMES[self.desc.table_kind]


def _plan_for(buffers: LatticeBuffers, info: dict) -> DecodePlan:
    layout, meta, freq = buffers.layout, buffers.stream_meta, buffers.freq_tables
    device = meta.device
    key = (meta.data_ptr(), freq.data_ptr(), device, FORCE_TABLE_KIND)
    plan = getattr(layout, "_lattice_rans_hip_plan", None)
    if plan is not None and plan.key == key:
        return plan

    lib = _hip.library()
    meta_host = np.ascontiguousarray(meta.detach().cpu().numpy(), dtype=np.int32)      # one small D2H, first call only
    freq_host = np.ascontiguousarray(freq.detach().cpu().view(torch.int16).numpy()).view(np.uint16)
    if meta_host.shape != (17, 4):
        raise ValueError(f"lattice_rans stream_meta must be (17, 4), got {meta_host.shape}")
    desc = _hip.PlanDesc()
    caps = _hip.device_info(device.index if device.index is not None else torch.cuda.current_device())
    status = lib.ep_hip_plan_describe(
        meta_host.ctypes.data, freq_host.ctypes.data if freq_host.size else None, freq_host.size, info["prob_bits"],
        info["tile_elements"], caps.lds_bytes_per_block, -1 if FORCE_TABLE_KIND is None else FORCE_TABLE_KIND, ctypes.byref(desc))
    if status == _hip.EINVAL:
        raise ValueError("lattice_rans stream_meta / freq_tables are inconsistent (ranges, sums or coset stream)")
    _hip.check("ep_hip_plan_describe", status)
    tables = torch.empty(desc.table_bytes, dtype=torch.uint8, device=device)
    error = torch.zeros(1, dtype=torch.int32, device=device)
    _hip.check("ep_hip_plan_build", lib.ep_hip_plan_build(
        meta.data_ptr(), _hip.pointer(freq), ctypes.byref(desc), tables.data_ptr(), _hip.current_stream(device)))
    plan = DecodePlan(desc=desc, tables=tables, error=error, key=key)
    layout._lattice_rans_hip_plan = plan
    return plan


def decode(buffers: LatticeBuffers, *, shape, dtype, threads_per_block=None, l2_prefetch=True) -> torch.Tensor:
    payload = buffers.payload
    device = payload.device
    if device.type != "cuda":
        raise RuntimeError(f"the hip lane decodes device buffers only, got {device}")
    info = decode_geometry(buffers._asdict(), shape)
    rows, cols = info["rows"], info["cols"]
    if buffers.scales.numel() != rows or buffers.states.numel() != max(1, info["total_tiles"]) * 32 \
            or buffers.offsets.numel() != max(1, info["total_tiles"]) + 1:
        raise ValueError("lattice_rans buffers do not match the container geometry")
    for tensor in buffers:
        if not tensor.is_contiguous():
            raise ValueError("lattice_rans buffers must be contiguous")
    via_float32 = dtype in _VIA_FLOAT32
    out_dtype = torch.float32 if via_float32 else dtype
    if out_dtype not in _hip.STORE_KINDS:
        raise ValueError(f"lattice_rans does not support output dtype {dtype}")
    with torch.cuda.device(device):
        plan = _plan_for(buffers, info)
        out = torch.empty((rows, cols), dtype=out_dtype, device=device)
        _hip.check("ep_hip_decode_lattice", _hip.library().ep_hip_decode_lattice(
            _hip.pointer(payload), payload.numel(), buffers.offsets.data_ptr(), buffers.states.data_ptr(),
            buffers.scales.data_ptr(), plan.tables.data_ptr(), ctypes.byref(plan.desc), out.data_ptr(),
            _hip.STORE_KINDS[out_dtype], rows, cols, info["tile_elements"], plan.error.data_ptr(),
            _hip.current_stream(device)))
    return snap_to_container(out, dtype) if via_float32 else out


def plan_of(buffers: LatticeBuffers) -> DecodePlan | None:
    """The cached plan of a container that has been decoded at least once."""
    return getattr(buffers.layout, "_lattice_rans_hip_plan", None)


def check_errors(buffers: LatticeBuffers) -> None:
    """Synchronises and raises ValueError if any decode of this container flagged a corrupt stream.

    The reference passes an error word to its kernels and never reads it (cuda.py:756,765,773); here it can be read
    on demand, off the hot path.
    """
    plan = plan_of(buffers)
    if plan is None:
        return
    code = int(plan.error.item())
    if code:
        plan.error.zero_()
        raise ValueError(f"lattice_rans decode error {code}: {_hip.DECODE_ERRORS.get(code, 'unknown')}")


def encode(**kwargs):
    """Encoding is CPU work in this package; the scheme routes it to the eager lane."""
    from . import eager
    weight = kwargs.pop("weight")
    device = weight.device
    packed = eager.encode(weight=weight.cpu(), **kwargs)
    return LatticeBuffers._make(value.to(device) for value in packed)
