"""`hip` lane of tile_ans: lossless decode on an MI355X through ep_hip_decode_tile_ans, and encode of device tensors.

Lane contract of the reference's CUDA lane (entropack/schemes/tile_ans/cuda.py:117-170): buffers on the device, the
result a flat tensor of `dtype` on the same device, enqueued on torch's current stream without a host
synchronisation. The lane modes are read back once per container and kept on the layout tensor object, as there.
There is no CPU path in this module and no fallback.
"""
import ctypes

import numpy as np
import torch

from ...backends import hip as _hip
from .format import LANE_ANS, LANE_RAW, NUM_STATES, TileBuffers, lane_modes_cached, make_layout, num_tiles, parse_layout_cached


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


def encode(*, weight: torch.Tensor, tile_elements: int, probability_bits: int, raw_lane_threshold: float, **_ignored) -> TileBuffers:
    """Lane contract of the reference's CUDA lane (entropack/schemes/tile_ans/cuda.py:64-119): the tensor is on the device
    and so are the buffers returned. Byte histograms, stream coding, cumulative sum and gather are kernels
    (`ep_hip_tile_ans_histogram`, `ep_hip_tile_ans_encode`, `ep_hip_encode_offsets`, `ep_hip_encode_gather`); the
    decisions in between (precision, tables, raw or coded per lane) are the CPU lane's own code on 256 counts per byte
    lane, so the container is byte-identical to the CPU lane's."""
    from ..lattice_rans.hip_encode import table_entries
    from . import eager
    if weight.numel() == 0:
        raise ValueError("tile_ans does not support empty tensors")
    if weight.device.type != "cuda":
        raise ValueError("the hip lane encodes tensors that are on the GPU; use execution_backend='eager' for CPU tensors")
    device = weight.device
    contiguous = weight.detach().contiguous()
    if contiguous.data_ptr() % 16:
        contiguous = contiguous.clone()
    num_elements, num_lanes = contiguous.numel(), contiguous.element_size()
    if num_lanes not in (1, 2, 4, 8):
        raise ValueError(f"tile_ans on the device takes elements of 1, 2, 4 or 8 bytes, got {num_lanes}")
    lib, stream = _hip.library(), _hip.current_stream(device)
    counts_device = torch.empty((num_lanes, 256), dtype=torch.int64, device=device)
    _hip.check("ep_hip_tile_ans_histogram", lib.ep_hip_tile_ans_histogram(
        contiguous.data_ptr(), num_elements, num_lanes, counts_device.data_ptr(), stream))
    counts = counts_device.cpu().numpy()
    probability_bits, freq, cdfs, tables, modes = eager.coding_plan(counts, probability_bits, raw_lane_threshold, tile_elements)

    tiles = num_tiles(num_elements, tile_elements)
    streams = tiles * num_lanes
    coded = int((modes == LANE_ANS).sum())
    entries = table_entries(freq.astype(np.int64).reshape(-1), cdfs.astype(np.int64).reshape(-1)).to(device)
    raw_flags = np.ascontiguousarray(modes == LANE_RAW, dtype=np.uint8)
    states = torch.empty((tiles * coded, NUM_STATES), dtype=torch.int32, device=device)
    stream_words = torch.empty(streams, dtype=torch.int32, device=device)
    scratch = torch.empty(streams * tile_elements, dtype=torch.int16, device=device)
    error = torch.zeros(1, dtype=torch.int32, device=device)
    offsets = torch.empty(streams + 1, dtype=torch.int32, device=device)
    total = torch.empty(1, dtype=torch.int64, device=device)
    _hip.check("ep_hip_tile_ans_encode", lib.ep_hip_tile_ans_encode(
        contiguous.data_ptr(), num_elements, num_lanes, tile_elements, probability_bits, entries.data_ptr(), raw_flags.ctypes.data,
        states.data_ptr() if coded else 0, stream_words.data_ptr(), scratch.data_ptr(), tile_elements, error.data_ptr(), stream))
    _hip.check("ep_hip_encode_offsets", lib.ep_hip_encode_offsets(stream_words.data_ptr(), streams, offsets.data_ptr(), total.data_ptr(), stream))
    words = int(total.item())
    if int(error.item()):
        raise RuntimeError("tile_ans device encode met a symbol its frequency table does not hold")
    if words >= 1 << 32:
        raise ValueError("tile_ans payload exceeds uint32 offset capacity")
    payload = torch.empty(words, dtype=torch.int16, device=device)
    if words:
        _hip.check("ep_hip_encode_gather", lib.ep_hip_encode_gather(
            scratch.data_ptr(), offsets.data_ptr(), streams, tile_elements, payload.data_ptr(), stream))
    return TileBuffers(
        payload=payload.view(torch.uint16), offsets=offsets.view(torch.uint32), states=states.view(torch.uint32),
        decode_tables=eager.as_unsigned_tensor(tables, np.int32).to(device),
        lane_modes=torch.from_numpy(np.ascontiguousarray(modes, dtype=np.uint8)).to(device),
        layout=make_layout(num_elements, num_lanes, tile_elements, probability_bits).to(device),
    )
