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

from ..base import cached_parse, host_copy
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
    tile_elements, prob_bits, num_lanes, num_elements = (int(v) for v in host_copy(layout).tolist())
    if tile_elements <= 0 or prob_bits not in SUPPORTED_PROB_BITS or num_lanes <= 0 or num_elements <= 0:
        raise ValueError(f"invalid tile_ans layout values: tile_elements={tile_elements}, prob_bits={prob_bits}, "
                         f"num_lanes={num_lanes}, num_elements={num_elements}")
    return tile_elements, prob_bits, num_lanes, num_elements


def parse_layout_cached(layout: torch.Tensor) -> tuple[int, int, int, int]:
    return cached_parse(layout, parse_layout, "_tile_ans_layout")


def lane_modes_cached(buffers: "TileBuffers") -> tuple[int, ...]:
    """The lane modes as Python ints, read from the device once per container (kept on the layout tensor object)."""
    return cached_parse(buffers.layout, lambda _: tuple(int(v) for v in host_copy(buffers.lane_modes).tolist()),
                        "_tile_ans_lane_modes")


def _stream_lengths(offsets: torch.Tensor, lane: int, tiles: int) -> torch.Tensor:
    """Words of each of a byte lane's `tiles` streams."""
    begin = lane * tiles
    return offsets[begin + 1:begin + tiles + 1] - offsets[begin:begin + tiles]


def validate_packed(buffers: dict, shape, dtype: torch.dtype) -> None:
    """Everything that can be told about a container without decoding it: the six tensors exist with their dtypes and
    ranks on one device, the layout matches `shape` / `dtype`, every table, state and offset array has the size the
    layout implies, offsets cover the payload monotonically, raw streams have exactly their tiles' bytes.
    Same checks and exception types as the reference's (schemes/tile_ans/format.py:96-164)."""
    absent = sorted(set(PACKED_KEYS) - set(buffers))
    if absent:
        raise ValueError(f"tile_ans container lacks buffers {absent}")
    held = {key: buffers[key] for key in PACKED_KEYS}
    strangers = [key for key, value in held.items() if not isinstance(value, torch.Tensor)]
    if strangers:
        raise TypeError(f"tile_ans buffers must be tensors; {strangers} are not")
    for key, tensor in held.items():
        wanted_dtype, wanted_rank = BUFFER_LAYOUT[key]
        if (tensor.dtype, tensor.ndim) != (wanted_dtype, wanted_rank):
            raise ValueError(f"tile_ans buffer '{key}' must be {wanted_dtype} of rank {wanted_rank}, got {tensor.dtype} of shape {tuple(tensor.shape)}")
        if not tensor.is_contiguous():
            raise ValueError(f"tile_ans buffer '{key}' must be contiguous")
    if len({tensor.device for tensor in held.values()}) > 1:
        raise ValueError(f"tile_ans buffers sit on different devices: { {key: str(t.device) for key, t in held.items()} }")

    tile_elements, prob_bits, num_lanes, num_elements = parse_layout(held["layout"])
    dims = tuple(shape)
    if not all(isinstance(dim, int) and dim >= 0 for dim in dims):
        raise ValueError(f"tile_ans tensor shape {dims} is not a tuple of sizes")
    if math.prod(dims) != num_elements:
        raise ValueError(f"tile_ans container holds {num_elements} elements, shape {dims} asks for {math.prod(dims)}")
    width = torch.empty((), dtype=dtype).element_size()
    if width != num_lanes:
        raise ValueError(f"tile_ans container has {num_lanes} byte lanes, {dtype} elements have {width} bytes")

    tiles = num_tiles(num_elements, tile_elements)
    modes = held["lane_modes"].detach().cpu().tolist()
    if len(modes) != num_lanes or any(mode not in (LANE_ANS, LANE_RAW) for mode in modes):
        raise ValueError(f"tile_ans lane_modes must be {num_lanes} values of {LANE_ANS} (coded) or {LANE_RAW} (raw), got {modes}")
    sizes = {
        "decode_tables": (num_lanes, 1 << prob_bits),
        "states": (tiles * modes.count(LANE_ANS), NUM_STATES),
        "offsets": (tiles * num_lanes + 1,),
    }
    for key, wanted in sizes.items():
        if tuple(held[key].shape) != wanted:
            raise ValueError(f"tile_ans buffer '{key}' must have shape {wanted} for this layout, got {tuple(held[key].shape)}")

    offsets = held["offsets"].detach().cpu().to(torch.int64)
    if int(offsets[0]) != 0 or int(offsets[-1]) != held["payload"].numel() or bool((offsets.diff() < 0).any()):
        raise ValueError("tile_ans offsets must rise from 0 to the payload length")
    tail = num_elements - (tiles - 1) * tile_elements
    for lane, mode in enumerate(modes):
        if mode == LANE_RAW:
            expect = [(tile_elements + 1) // 2] * (tiles - 1) + [(tail + 1) // 2]
            if _stream_lengths(offsets, lane, tiles).tolist() != expect:
                raise ValueError(f"tile_ans raw lane {lane} does not hold exactly its tiles' bytes")
