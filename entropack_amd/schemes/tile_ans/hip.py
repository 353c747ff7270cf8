"""`hip` lane of tile_ans: lossless decode on an MI355X through ep_hip_decode_tile_ans.

Lane contract of the reference's CUDA lane (entropack/schemes/tile_ans/cuda.py:117-170): buffers on the device, the
result a flat tensor of `dtype` on the same device, enqueued on torch's current stream without a host
synchronisation. The lane modes are read back once per container and kept on the layout tensor object, as there.
There is no CPU path in this module and no fallback.
"""
import ctypes

import numpy as np
import torch

from ...backends import hip as _hip
from .format import TileBuffers, lane_modes_cached, num_tiles, parse_layout_cached


def _error_word(buffers: TileBuffers) -> torch.Tensor:
    word = getattr(buffers.layout, "_tile_ans_hip_error", None)
    if word is None or word.device != buffers.payload.device:
        word = torch.zeros(1, dtype=torch.int32, device=buffers.payload.device)
        buffers.layout._tile_ans_hip_error = word
    return word


def decode(buffers: TileBuffers, *, dtype: torch.dtype, threads_per_block=None) -> torch.Tensor:
    device = buffers.payload.device
    if device.type != "cuda":
        raise RuntimeError(f"the hip lane decodes device buffers only, got {device}")
    tile_elements, prob_bits, num_lanes, num_elements = parse_layout_cached(buffers.layout)
    if torch.empty((), dtype=dtype).element_size() != num_lanes:
        raise ValueError(f"tile_ans layout has {num_lanes} byte lanes but dtype {dtype} has another width")
    modes = lane_modes_cached(buffers)
    tiles = num_tiles(num_elements, tile_elements)
    coded = sum(1 for mode in modes if mode == 0)
    if len(modes) != num_lanes or buffers.offsets.numel() != tiles * num_lanes + 1 or buffers.states.numel() != tiles * coded * 32 \
            or tuple(buffers.decode_tables.shape) != (num_lanes, 1 << prob_bits):
        raise ValueError("tile_ans buffers do not match the container layout")
    for tensor in buffers:
        if not tensor.is_contiguous():
            raise ValueError("tile_ans buffers must be contiguous")
    modes_host = np.asarray(modes, dtype=np.uint8)
    with torch.cuda.device(device):
        out = torch.empty(num_elements * num_lanes, dtype=torch.uint8, device=device)
        _hip.check("ep_hip_decode_tile_ans", _hip.library().ep_hip_decode_tile_ans(
            _hip.pointer(buffers.payload), buffers.payload.numel(), buffers.offsets.data_ptr(), _hip.pointer(buffers.states),
            buffers.decode_tables.data_ptr(), modes_host.ctypes.data, tile_elements, prob_bits, num_lanes, num_elements,
            out.data_ptr(), _error_word(buffers).data_ptr(), _hip.current_stream(device)))
    return out.view(dtype)


def check_errors(buffers: TileBuffers) -> None:
    """Synchronises and raises ValueError if any decode of this container flagged a corrupt stream."""
    word = getattr(buffers.layout, "_tile_ans_hip_error", None)
    if word is None:
        return
    code = int(word.item())
    if code:
        word.zero_()
        raise ValueError(f"tile_ans decode error {code}: {_hip.DECODE_ERRORS.get(code, 'unknown')}")


def encode(**kwargs):
    """Encoding is CPU work in this package; the scheme routes it to the eager lane."""
    from . import eager
    weight = kwargs.pop("weight")
    device = weight.device
    packed = eager.encode(weight=weight.cpu(), **kwargs)
    return TileBuffers._make(value.to(device) for value in packed)
