"""On-disk/in-memory format of a `lattice_rans` container, and its config.

A container is seven buffers (entropack/schemes/lattice_rans/format.py:70-101 of the reference):

    payload      u16[W]      renormalisation words of all tiles, tile after tile
    offsets      u32[T + 1]  first word of each tile (offsets[T] == W)
    states       u32[T, 32]  final encoder states = initial decoder states
    stream_meta  i32[17, 4]  per stream: n_symbols, sym_min, freq_offset, alphabet
    freq_tables  u16[sum A]  normalised frequencies, stream after stream; each stream sums to 2**prob_bits
    scales       f32[rows]   reconstruction scale of each row
    layout       i64[3]      padded cols, prob_bits, tile_elements

Stream 0 codes the coset bit of each 8-vector; stream 1 + 2f + c codes field f of coset-c vectors. A tile covers
`tile_vectors = max(32, tile_elements // 9)` consecutive vectors and is decoded by 32 interleaved rANS lanes.
"""
import logging
from dataclasses import dataclass
from typing import Annotated, NamedTuple

import torch

from ..base import cached_parse, host_copy
from ..config import CompressionConfig, OneOf, Range

log = logging.getLogger("entropack.lattice_rans")

LATTICE_DIM = 8
NUM_FIELDS = 8
NUM_STREAMS = 1 + 2 * NUM_FIELDS
NUM_STATES = 32
STATE_MIN = 1 << 15
SUPPORTED_PROB_BITS = (9, 10, 11, 12, 13, 14, 15)
META_WIDTH = 4
META_N_SYMBOLS, META_SYM_MIN, META_FREQ_OFFSET, META_ALPHABET = range(4)

SUPPORTED_DTYPES = (
    torch.float32, torch.float16, torch.bfloat16,
    torch.float8_e4m3fn, torch.float8_e4m3fnuz, torch.float8_e5m2, torch.float8_e5m2fnuz,
    torch.int64, torch.int32, torch.int16, torch.int8, torch.uint64, torch.uint32, torch.uint16, torch.uint8, torch.bool,
)
INTEGER_DTYPES = frozenset({
    torch.int64, torch.int32, torch.int16, torch.int8, torch.uint64, torch.uint32, torch.uint16, torch.uint8,
})
BUFFER_DTYPES = {
    "payload": torch.uint16, "offsets": torch.uint32, "states": torch.uint32, "stream_meta": torch.int32,
    "freq_tables": torch.uint16, "scales": torch.float32, "layout": torch.int64,
}


@dataclass
class EntroPackLossyConfig(CompressionConfig):
    """Lossy E8-lattice + rANS compression of finite 2-D tensors.

    Only `execution_backend` matters when decoding; tile size and probability precision travel with the container.
    Field names, defaults and ranges are those of the reference (format.py:25-51).
    """

    #: Requested bits per element, in [0.001, 11]; capped at the input's own width.
    target_bpp: Annotated[float, Range(0.001, 11.0)] = 4.0
    #: rANS probability precision; None or 0 = choose (11 up to 7 bpp, else 12, growing when an alphabet needs it).
    prob_bits: Annotated[int | None, OneOf(SUPPORTED_PROB_BITS, silent=(0,))] = None
    #: Symbols per tile; None = choose from the target rate.
    tile_elements: Annotated[int | None, Range(1, None)] = None
    #: Per-row rate-distortion sweeps (encoder); 0 = off.
    row_rdo_iterations: Annotated[int, Range(0, 8)] = 0
    #: Candidate scales per row for those sweeps.
    row_rdo_candidates: Annotated[int, Range(1, None)] = 5
    #: Bisection steps of the scale search.
    scale_search_iterations: Annotated[int, Range(1, None)] = 12
    #: Vectors sampled by the scale search.
    scale_search_max_vectors: Annotated[int, Range(1, None)] = 262144
    #: Accepted for compatibility; the HIP kernels size their own workgroups.
    threads_per_block: Annotated[int | None, Range(1, None)] = None
    #: Accepted for compatibility; the HIP kernels always stream the payload ahead of use.
    l2_prefetch: bool = True


LatticeRANSConfig = EntroPackLossyConfig


class LatticeBuffers(NamedTuple):
    payload: torch.Tensor
    offsets: torch.Tensor
    states: torch.Tensor
    stream_meta: torch.Tensor
    freq_tables: torch.Tensor
    scales: torch.Tensor
    layout: torch.Tensor


PACKED_KEYS = LatticeBuffers._fields


def recommended_tile_elements(target_bpp: float) -> int:
    for limit, size in ((2.0, 32768), (4.0, 16384), (7.0, 8192)):
        if target_bpp <= limit:
            return size
    return 4096


def resolve_prob_bits(prob_bits, target_bpp: float) -> tuple[int, bool]:
    """(prob_bits, chosen automatically?)"""
    if prob_bits in (None, 0):
        return (12 if float(target_bpp) > 7.0 else 11), True
    return int(prob_bits), False


def vector_tile_elements(tile_elements: int) -> int:
    return max(32, int(tile_elements) // 9)


def make_layout(cols: int, prob_bits: int, tile_elements: int) -> torch.Tensor:
    return torch.tensor([cols, prob_bits, tile_elements], dtype=torch.int64)


def parse_layout(layout: torch.Tensor) -> dict:
    if layout.dtype != torch.int64 or layout.ndim != 1 or layout.numel() != 3:
        raise ValueError("lattice_rans layout must be int64[3]")
    cols, prob_bits, tile_elements = (int(v) for v in host_copy(layout).tolist())
    if cols <= 0 or cols % LATTICE_DIM:
        raise ValueError("lattice_rans vector-plane format requires positive cols divisible by 8")
    if prob_bits not in SUPPORTED_PROB_BITS:
        raise ValueError(f"lattice_rans prob_bits {prob_bits} unsupported")
    if tile_elements <= 0:
        raise ValueError("lattice_rans tile_elements must be positive")
    return {"cols": cols, "prob_bits": prob_bits, "tile_elements": tile_elements}


def decode_geometry(buffers: dict, shape) -> dict:
    """Everything a decoder needs to know about sizes; the layout tensor is parsed once and remembered on it."""
    stored = cached_parse(buffers["layout"], parse_layout, "_lattice_rans_layout")
    rows = int(shape[0])
    tile_vectors = vector_tile_elements(stored["tile_elements"])
    vectors = rows * (stored["cols"] // LATTICE_DIM)
    return {**stored, "rows": rows, "n_streams": NUM_STREAMS, "tile_vectors": tile_vectors, "vectors": vectors,
            "total_tiles": (vectors + tile_vectors - 1) // tile_vectors}


def snap_to_container(values: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Saturating cast of a float32 reconstruction into the container dtype (reference format.py:153-168)."""
    if dtype == torch.float32:
        return values
    if dtype == torch.bool:
        return values.round() != 0
    if dtype in INTEGER_DTYPES:
        info = torch.iinfo(dtype)
        top = torch.nextafter(torch.tensor(float(info.max) + 1.0, dtype=values.dtype), torch.tensor(float("-inf"), dtype=values.dtype))
        return values.round().clamp(float(info.min), float(top)).to(dtype)
    limit = float(torch.finfo(dtype).max)
    return values.clamp(-limit, limit).to(dtype)


def validate_packed(buffers: dict, shape, dtype: torch.dtype) -> dict:
    """Structural checks of a container (the invariants listed in the reference's format.py:192-312)."""
    missing = [key for key in PACKED_KEYS if key not in buffers]
    if missing:
        raise ValueError(f"lattice_rans packed data is missing buffers: {missing}")
    extra = sorted(set(buffers) - set(PACKED_KEYS))
    if extra:
        raise ValueError(f"lattice_rans packed data has unexpected buffers: {extra}")
    if dtype not in SUPPORTED_DTYPES:
        raise ValueError(f"lattice_rans does not support output dtype {dtype}")
    if len(shape) != 2 or any(not isinstance(d, int) or d <= 0 for d in shape):
        raise ValueError(f"lattice_rans shape must be non-empty 2D, got {tuple(shape)}")
    if len({buffers[key].device for key in PACKED_KEYS}) != 1:
        raise ValueError("lattice_rans packed buffers must share one device")
    for key, expected in BUFFER_DTYPES.items():
        if buffers[key].dtype != expected:
            raise ValueError(f"lattice_rans buffer '{key}' must be {expected}, got {buffers[key].dtype}")
        if not buffers[key].is_contiguous():
            raise ValueError(f"lattice_rans buffer '{key}' must be contiguous")
    info = decode_geometry(buffers, shape)
    rows, cols = shape
    if not 0 <= info["cols"] - cols < LATTICE_DIM:
        raise ValueError(f"lattice_rans layout columns {info['cols']} do not match {(rows, cols)}")
    scales = buffers["scales"]
    if scales.ndim != 1 or scales.numel() != rows:
        raise ValueError("lattice_rans scales must be 1D with one entry per row")
    if not bool((torch.isfinite(scales) & (scales > 0)).all()):
        raise ValueError("lattice_rans scales must be finite and positive")
    tiles = max(1, info["total_tiles"])
    if tuple(buffers["stream_meta"].shape) != (NUM_STREAMS, META_WIDTH):
        raise ValueError(f"lattice_rans stream_meta must be ({NUM_STREAMS},{META_WIDTH})")
    if tuple(buffers["states"].shape) != (tiles, NUM_STATES):
        raise ValueError("lattice_rans states shape does not match total_tiles")
    offsets = buffers["offsets"].to(torch.int64).cpu()
    if offsets.numel() != tiles + 1:
        raise ValueError("lattice_rans offsets length must be total_tiles+1")
    if int(offsets[0]) != 0 or int(offsets[-1]) != buffers["payload"].numel():
        raise ValueError("lattice_rans payload offsets endpoints are invalid")
    if bool((offsets[1:] < offsets[:-1]).any()):
        raise ValueError("lattice_rans payload offsets must be monotone")
    meta = buffers["stream_meta"].detach().cpu().to(torch.int64)
    freq = buffers["freq_tables"].detach().cpu().to(torch.int64)
    table_size = 1 << info["prob_bits"]
    cursor = 0
    for stream in range(NUM_STREAMS):
        n, _minimum, offset, alphabet = (int(v) for v in meta[stream])
        if n < 0 or alphabet < 0 or offset != cursor or offset + alphabet > freq.numel():
            raise ValueError("lattice_rans frequency-table ranges must be contiguous and non-negative")
        if (n == 0) != (alphabet == 0):
            raise ValueError("lattice_rans empty table metadata is inconsistent")
        if alphabet and (alphabet > table_size or int(freq[offset:offset + alphabet].sum()) != table_size):
            raise ValueError("lattice_rans normalized frequencies have an invalid sum")
        cursor += alphabet
    if cursor != freq.numel():
        raise ValueError("lattice_rans frequency table has trailing entries")
    counts = meta[:, META_N_SYMBOLS].tolist()
    if counts[0] != info["vectors"] or int(meta[0, META_SYM_MIN]) != 0:
        raise ValueError("lattice_rans coset table metadata is invalid")
    if counts[1] + counts[2] != info["vectors"] or any(
            counts[1 + 2 * f] != counts[1] or counts[2 + 2 * f] != counts[2] for f in range(NUM_FIELDS)):
        raise ValueError("lattice_rans conditioned table counts are inconsistent")
    return info
