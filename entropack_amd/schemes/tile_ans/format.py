"""On-disk/in-memory format of a `tile_ans` container (lossless), and its config.

Every element of the tensor is split into its bytes ("byte lanes", lane b = byte b of the element in memory order);
each lane is cut into tiles of `tile_elements` elements and each (lane, tile) pair is one stream, lane-major. A lane
is either stored raw (two bytes per 16-bit word, even element in the low byte) or entropy-coded with 32 interleaved
rANS states over one 256-symbol table per lane (entropack/schemes/tile_ans/format.py:53-59,
eager.py:145-228 of the reference):

    payload        u16[W]                    words of all streams, stream after stream
    offsets        u32[S + 1]                first word of each stream, S = lanes * tiles
    states         u32[tiles * A, 32]        final encoder states of the coded streams, A = coded lanes, lane-major
    decode_tables  u32[lanes, 2**prob_bits]  slot -> cdf << 20 | freq << 8 | symbol (freq 4096 stored as 0)
    lane_modes     u8[lanes]                 0 = coded, 1 = raw
    layout         i64[4]                    tile_elements, prob_bits, lanes, elements
"""
import math
from dataclasses import dataclass
from typing import Annotated, NamedTuple

import torch

from ..base import cached_parse
from ..config import CompressionConfig, OneOf, Range

AUTO_PROB_BITS = 0
AUTO_TILE_ELEMENTS = 0
SUPPORTED_PROB_BITS = (9, 10, 11, 12)
NUM_STATES = 32
STATE_MIN = 1 << 15
LANE_ANS, LANE_RAW = 0, 1
TILE_ELEMENTS_LIMIT = 1 << 31
FREQ_STORED_AS_ZERO = 4096


@dataclass
class TileANSConfig(CompressionConfig):
    """Lossless compression of any supported dtype. Field names, defaults and ranges are the reference's
    (format.py:33-47); tile size and probability precision travel with the container, 0 = choose."""

    #: Elements per independent tile; 0 = 4096, or 8192 for tensors above 32 MiB.
    tile_elements: Annotated[int, Range(0, TILE_ELEMENTS_LIMIT - 1,
                                        message="tile_elements must be positive, or 0 for automatic selection, "
                                                "and fit the CUDA int32 launch ABI")] = AUTO_TILE_ELEMENTS
    #: Probability-table precision; 0 = choose from the byte histograms.
    probability_bits: Annotated[int, OneOf(SUPPORTED_PROB_BITS, silent=(AUTO_PROB_BITS,))] = AUTO_PROB_BITS
    #: Byte lanes whose estimated cost reaches this many bits per symbol are stored raw.
    raw_lane_threshold: Annotated[float, Range(0.0, 8.0)] = 7.9
    #: Accepted for compatibility with the reference's GPU lanes; the kernels here choose their own launch shape.
    threads_per_block: Annotated[int | None, Range(1, None)] = None


#: dtype -> (tile_elements, probability_bits) a layer uses when given no config (format.py:50-58 of the reference).
OPTIONS_BY_DTYPE = {
    torch.float32: (8192, 10), torch.float16: (8192, 11), torch.bfloat16: (0, 11),
    torch.float8_e4m3fn: (8192, 0), torch.float8_e4m3fnuz: (8192, 0), torch.float8_e5m2: (8192, 0), torch.float8_e5m2fnuz: (8192, 0),
    torch.int64: (8192, 10), torch.int32: (16384, 10), torch.int16: (8192, 9), torch.int8: (8192, 0),
    torch.uint64: (8192, 9), torch.uint32: (8192, 10), torch.uint16: (8192, 9), torch.uint8: (8192, 0), torch.bool: (8192, 9),
}


class TileBuffers(NamedTuple):
    payload: torch.Tensor
    offsets: torch.Tensor
    states: torch.Tensor
    decode_tables: torch.Tensor
    lane_modes: torch.Tensor
    layout: torch.Tensor


PACKED_KEYS = TileBuffers._fields
BUFFER_LAYOUT = {
    "payload": (torch.uint16, 1), "offsets": (torch.uint32, 1), "states": (torch.uint32, 2),
    "decode_tables": (torch.uint32, 2), "lane_modes": (torch.uint8, 1), "layout": (torch.int64, 1),
}


def num_tiles(num_elements: int, tile_elements: int) -> int:
    return -(-num_elements // tile_elements)


def make_layout(num_elements: int, num_lanes: int, tile_elements: int, probability_bits: int) -> torch.Tensor:
    if probability_bits not in SUPPORTED_PROB_BITS:
        raise ValueError(f"probability_bits must be one of {SUPPORTED_PROB_BITS}")
    return torch.tensor([tile_elements, probability_bits, num_lanes, num_elements], dtype=torch.int64)


def parse_layout(layout: torch.Tensor) -> tuple[int, int, int, int]:
    """(tile_elements, prob_bits, lanes, elements)"""
    if layout.dtype != torch.int64 or layout.ndim != 1 or layout.numel() != 4:
        raise ValueError("tile_ans layout must be int64[4]")
    tile_elements, prob_bits, num_lanes, num_elements = (int(v) for v in layout.detach().cpu().tolist())
    if tile_elements <= 0 or prob_bits not in SUPPORTED_PROB_BITS or num_lanes <= 0 or num_elements <= 0:
        raise ValueError(f"invalid tile_ans layout values: tile_elements={tile_elements}, prob_bits={prob_bits}, "
                         f"num_lanes={num_lanes}, num_elements={num_elements}")
    return tile_elements, prob_bits, num_lanes, num_elements


def parse_layout_cached(layout: torch.Tensor) -> tuple[int, int, int, int]:
    return cached_parse(layout, parse_layout, "_tile_ans_layout")


def lane_modes_cached(buffers: "TileBuffers") -> tuple[int, ...]:
    """The lane modes as Python ints, read from the device once per container (kept on the layout tensor object)."""
    return cached_parse(buffers.layout, lambda _: tuple(int(v) for v in buffers.lane_modes.detach().cpu().tolist()),
                        "_tile_ans_lane_modes")


def validate_packed(buffers: dict, shape, dtype: torch.dtype) -> None:
    """Structural checks of a container, with the reference's messages (format.py:96-164)."""
    missing = [key for key in PACKED_KEYS if key not in buffers]
    if missing:
        raise ValueError(f"tile_ans packed data is missing buffers: {missing}")
    if not all(isinstance(buffers[key], torch.Tensor) for key in PACKED_KEYS):
        raise TypeError("tile_ans packed buffers must be torch.Tensor values")
    for key, (wanted, ndim) in BUFFER_LAYOUT.items():
        tensor = buffers[key]
        if not tensor.is_contiguous():
            raise ValueError(f"tile_ans buffer '{key}' must be contiguous")
        if tensor.dtype != wanted or tensor.ndim != ndim:
            raise ValueError(f"tile_ans buffer '{key}' must be {ndim}D {wanted}, got shape={tuple(tensor.shape)}, dtype={tensor.dtype}")
    devices = {buffers[key].device for key in PACKED_KEYS}
    if len(devices) != 1:
        raise ValueError(f"tile_ans packed buffers must share one device, got {devices}")

    tile_elements, prob_bits, num_lanes, num_elements = parse_layout(buffers["layout"])
    element_size = torch.empty((), dtype=dtype).element_size()
    if num_lanes != element_size:
        raise ValueError(f"tile_ans layout has {num_lanes} byte lanes but dtype {dtype} uses {element_size} bytes")
    shape = tuple(shape)
    if any(not isinstance(dim, int) or dim < 0 for dim in shape):
        raise ValueError(f"invalid tile_ans tensor shape: {shape}")
    if math.prod(shape) != num_elements:
        raise ValueError(f"tile_ans shape {shape} does not match {num_elements} elements")

    tiles = num_tiles(num_elements, tile_elements)
    streams = tiles * num_lanes
    if tuple(buffers["decode_tables"].shape) != (num_lanes, 1 << prob_bits):
        raise ValueError("tile_ans decode_tables shape does not match layout")
    if buffers["lane_modes"].numel() != num_lanes:
        raise ValueError("tile_ans lane_modes length does not match layout")
    modes = buffers["lane_modes"].detach().cpu()
    if ((modes != LANE_ANS) & (modes != LANE_RAW)).any():
        raise ValueError("tile_ans lane_modes contains an unknown codec mode")
    coded = int((modes == LANE_ANS).sum())
    if tuple(buffers["states"].shape) != (tiles * coded, NUM_STATES):
        raise ValueError("tile_ans states shape does not match ANS lanes/layout")
    if buffers["offsets"].numel() != streams + 1:
        raise ValueError("tile_ans offsets length does not match layout")
    offsets = buffers["offsets"].detach().cpu().to(torch.int64)
    if offsets[0] != 0 or offsets[-1] != buffers["payload"].numel():
        raise ValueError("tile_ans offsets endpoints are invalid")
    if (offsets[1:] < offsets[:-1]).any():
        raise ValueError("tile_ans offsets must be monotone")
    last = num_elements - (tiles - 1) * tile_elements
    for lane, mode in enumerate(modes.tolist()):
        if mode != LANE_RAW:
            continue
        sizes = offsets[lane * tiles + 1: (lane + 1) * tiles + 1] - offsets[lane * tiles: (lane + 1) * tiles]
        wanted = torch.full_like(sizes, (tile_elements + 1) // 2)
        wanted[-1] = (last + 1) // 2
        if not torch.equal(sizes, wanted):
            raise ValueError("tile_ans raw lane payload length is invalid")
