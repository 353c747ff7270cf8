"""CPU encoder of `tile_ans` (the `eager` lane; tensors on an MI355X are encoded there by the `hip` lane with this
module's decisions). There is no CPU decoder in this package.

Bit-identical to the reference's encoder (entropack/schemes/tile_ans/eager.py:17-228): same frequency normalisation
(largest-remainder with the same tie order), same lane-mode and probability-precision choice, same stream layout.
Histograms and table logic are numpy; the per-symbol rANS loop runs in libentropack_host.so (hc_tile_ans_encode).
"""
import ctypes

import numpy as np
import torch

from ..lattice_rans.eager import _threads, host_library
from .format import (
    AUTO_PROB_BITS, FREQ_STORED_AS_ZERO, LANE_ANS, LANE_RAW, NUM_STATES, SUPPORTED_PROB_BITS, TileBuffers, make_layout,
    num_tiles,
)

#: Precision choice: among tables whose estimated size is within this fraction of the input of the cheapest, the coarsest.
AUTO_RATIO_TOLERANCE = 0.0015


def normalize_counts(counts: np.ndarray, table_size: int) -> np.ndarray:
    """Frequencies summing to `table_size`, every occurring symbol at least 1.

    Floor of the exact share, then the deficit goes one unit at a time to the symbol with the largest remainder (a
    symbol's remainder drops by one when it is served; ties go to the smaller symbol); a surplus is taken one unit at
    a time from the symbol with the smallest remainder among those above 1 (its remainder rises by one). The loop is
    hc_tile_ans_normalize_counts of libentropack_host.so.
    """
    counts = np.ascontiguousarray(counts, dtype=np.int64)
    freq = np.empty(counts.size, dtype=np.uint16)
    status = host_library().hc_tile_ans_normalize_counts(counts.ctypes.data, counts.size, table_size, freq.ctypes.data)
    if status == -1:
        raise ValueError("cannot build an rANS codebook from empty input")
    if status == -3:
        raise MemoryError("frequency normalisation ran out of memory")
    if status != 0:
        raise ValueError("unable to normalize rANS frequencies")
    return freq


def tables_from_frequencies(frequencies: np.ndarray, probability_bits: int):
    """(cdf u16[lanes, 256], decode table u32[lanes, 2**pb]) of normalised frequencies."""
    frequencies = np.asarray(frequencies, dtype=np.uint16)
    table_size = 1 << probability_bits
    wide = frequencies.astype(np.int64)
    ends = np.cumsum(wide, axis=1)
    if not np.all(ends[:, -1] == table_size):
        raise AssertionError(f"normalized frequency sums are {ends[:, -1]}, expected {table_size}")
    starts = ends - wide
    tables = np.empty((frequencies.shape[0], table_size), dtype=np.uint32)
    symbols = np.arange(256, dtype=np.int64)
    for lane in range(frequencies.shape[0]):
        stored = np.where(wide[lane] == FREQ_STORED_AS_ZERO, 0, wide[lane])
        entry = (starts[lane] << 20) | (stored << 8) | symbols
        tables[lane] = np.repeat(entry, wide[lane]).astype(np.uint32)
    return starts.astype(np.uint16), tables


def _coded_bits(counts: np.ndarray, freq: np.ndarray, probability_bits: int) -> float:
    seen = counts > 0
    return float(np.sum(counts[seen].astype(np.float64) * (probability_bits - np.log2(freq[seen].astype(np.float64)))))


def lane_modes_from_counts(counts_by_lane, raw_lane_threshold: float, tile_elements: int, frequencies=None,
                           probability_bits: int | None = None) -> np.ndarray:
    """Raw or coded, per byte lane: raw when the (ideal, or table-quantised) cost per symbol reaches the threshold,
    which is first lowered by what the 32 states of a tile cost."""
    if not 0.0 <= raw_lane_threshold <= 8.0:
        raise ValueError("raw_lane_threshold must be in [0, 8]")
    limit = min(raw_lane_threshold, 8.0 - (NUM_STATES * 32) / tile_elements)
    counts_by_lane = np.asarray(counts_by_lane, dtype=np.int64)
    modes = np.empty(counts_by_lane.shape[0], dtype=np.uint8)
    for lane, counts in enumerate(counts_by_lane):
        total = int(counts.sum())
        if frequencies is None:
            p = counts[counts > 0].astype(np.float64) / total
            bits = -np.sum(p * np.log2(p))
        else:
            if probability_bits is None:
                raise ValueError("probability_bits is required with normalized frequencies")
            bits = _coded_bits(counts, frequencies[lane], probability_bits) / total
        modes[lane] = LANE_RAW if bits >= limit else LANE_ANS
    return modes


def select_coding_options(counts_by_lane, raw_lane_threshold: float, tile_elements: int):
    """Probability precision, tables and lane modes for `probability_bits = 0`: price every supported precision with
    the container's byte model and keep the coarsest one within tolerance of the cheapest."""
    counts_by_lane = np.asarray(counts_by_lane, dtype=np.int64)
    num_elements = int(counts_by_lane[0].sum())
    num_lanes = counts_by_lane.shape[0]
    tiles = num_tiles(num_elements, tile_elements)
    whole, tail = divmod(num_elements, tile_elements)
    raw_words = whole * ((tile_elements + 1) // 2) + (tail + 1) // 2
    ideal = lane_modes_from_counts(counts_by_lane, raw_lane_threshold, tile_elements)
    # A quantised table only adds cost: lanes raw at their entropy are raw at every precision.
    variants = SUPPORTED_PROB_BITS[:1] if np.all(ideal == LANE_RAW) else SUPPORTED_PROB_BITS
    priced = []
    for bits in variants:
        size = 1 << bits
        freq = np.stack([normalize_counts(counts, size) for counts in counts_by_lane])
        modes = lane_modes_from_counts(counts_by_lane, raw_lane_threshold, tile_elements, freq, bits)
        total = (tiles * num_lanes + 1) * 4 + num_lanes * size * 4 + num_lanes + 5 * 8
        for lane, mode in enumerate(modes):
            if mode == LANE_RAW:
                total += raw_words * 2
            else:
                total += _coded_bits(counts_by_lane[lane], freq[lane], bits) / 8
                total += tiles * NUM_STATES * 4
        priced.append((total, bits, freq, modes))
    slack = num_elements * num_lanes * AUTO_RATIO_TOLERANCE
    cheapest = min(entry[0] for entry in priced)
    _, bits, freq, modes = min((entry for entry in priced if entry[0] <= cheapest + slack), key=lambda entry: entry[1])
    cdfs, tables = tables_from_frequencies(freq, bits)
    return bits, freq, cdfs, tables, modes


def coding_plan(counts: np.ndarray, probability_bits: int, raw_lane_threshold: float, tile_elements: int):
    """(probability_bits, frequencies, cdfs, decode tables, lane modes) from the byte histograms int64[lanes, 256]: the
    whole of the encoder's decisions; what remains is the coding of the streams (both lanes of this package share it)."""
    if probability_bits == AUTO_PROB_BITS:
        return select_coding_options(counts, raw_lane_threshold, tile_elements)
    freq = np.stack([normalize_counts(c, 1 << probability_bits) for c in counts])
    cdfs, tables = tables_from_frequencies(freq, probability_bits)
    return probability_bits, freq, cdfs, tables, lane_modes_from_counts(counts, raw_lane_threshold, tile_elements)


def as_unsigned_tensor(array: np.ndarray, kind) -> torch.Tensor:
    """A numpy unsigned array as the torch tensor of the same unsigned dtype (through the signed view `kind`)."""
    return torch.from_numpy(array.view(kind)).view({np.int16: torch.uint16, np.int32: torch.uint32}[kind])


def encode(*, weight: torch.Tensor, tile_elements: int, probability_bits: int, raw_lane_threshold: float, **_ignored) -> TileBuffers:
    if weight.numel() == 0:
        raise ValueError("tile_ans does not support empty tensors")
    contiguous = weight.detach().contiguous().cpu()
    num_elements = contiguous.numel()
    num_lanes = contiguous.element_size()
    raw = np.ascontiguousarray(contiguous.reshape(-1).view(torch.uint8).numpy())
    by_lane = raw.reshape(num_elements, num_lanes)
    counts = np.stack([np.bincount(by_lane[:, lane], minlength=256) for lane in range(num_lanes)])
    probability_bits, freq, cdfs, tables, modes = coding_plan(counts, probability_bits, raw_lane_threshold, tile_elements)

    tiles = num_tiles(num_elements, tile_elements)
    coded = int((modes == LANE_ANS).sum())
    states = np.empty((tiles * coded, NUM_STATES), dtype=np.uint32)
    offsets = np.empty(tiles * num_lanes + 1, dtype=np.uint32)
    freq16 = np.ascontiguousarray(freq, dtype=np.uint16)
    cdf16 = np.ascontiguousarray(cdfs, dtype=np.uint16)
    raw_flags = np.ascontiguousarray(modes == LANE_RAW, dtype=np.uint8)
    words = ctypes.c_void_p()
    lib = host_library()
    status = lib.hc_tile_ans_encode(raw.ctypes.data, num_elements, num_lanes, tile_elements, probability_bits, freq16.ctypes.data,
                                    cdf16.ctypes.data, raw_flags.ctypes.data, states.ctypes.data, offsets.ctypes.data,
                                    ctypes.byref(words), _threads())
    if status == -2:
        raise ValueError("tile_ans payload exceeds uint32 offset capacity")
    if status != 0:
        raise MemoryError("tile_ans encoder ran out of memory")
    try:
        total = int(offsets[-1])
        payload = np.ctypeslib.as_array(ctypes.cast(words, ctypes.POINTER(ctypes.c_uint16)), shape=(max(total, 1),))[:total].copy()
    finally:
        lib.hc_free(words)
    as_torch = as_unsigned_tensor
    return TileBuffers(
        payload=as_torch(payload, np.int16), offsets=as_torch(offsets, np.int32), states=as_torch(states, np.int32),
        decode_tables=as_torch(tables, np.int32), lane_modes=torch.from_numpy(np.ascontiguousarray(modes, dtype=np.uint8)),
        layout=make_layout(num_elements, num_lanes, tile_elements, probability_bits),
    )


def decode(*_args, **_kwargs):
    raise RuntimeError("this package has no CPU decoder: tile_ans containers are decoded by the hip backend only")
