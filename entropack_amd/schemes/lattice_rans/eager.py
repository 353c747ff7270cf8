"""`eager` (CPU) lane of lattice_rans: the encoder.

CPU tensors are encoded here (tensors on an MI355X by the `hip` lane, with this module's orchestration). It restates the
reference's CPU encoder (entropack/schemes/lattice_rans/eager.py:91-341 and rans.py:12-95,133-258) so that the same
input and config give the same container, bit for bit: row RMS normalisation, a bisection of the lattice scale
against an analytic size model on a seeded row subsample, nearest-E8 quantisation, least-squares refit of the row
scales, Hamilton-normalised frequency tables and the tiled 32-way interleaved rANS encode. The per-vector and
per-symbol loops run in libentropack_host.so (csrc/host_codec.c).

The optional per-row rate-distortion pass (`row_rdo_iterations > 0`) is rdo.py.

`decode` is deliberately absent: containers are decoded by the `hip` lane. Asking this lane to decode raises.
"""
import ctypes
import math
import os

import numpy as np
import torch

from .format import (
    LATTICE_DIM, META_ALPHABET, META_FREQ_OFFSET, META_N_SYMBOLS, META_SYM_MIN, META_WIDTH, NUM_FIELDS, NUM_STATES,
    NUM_STREAMS, LatticeBuffers, log, make_layout, resolve_prob_bits, vector_tile_elements,
)

MIN_RMS = 1.0e-12
ALPHABET_COARSEN_MARGIN = 1.05
SUBSAMPLE_SEED_MULTIPLIER = 1000003
#: Constants of the analytic size model; they are part of what the scale search converges to.
MODEL_LAYOUT_BYTES = 64
MODEL_STREAM_META_BYTES = 408
MODEL_SLACK_BYTES = 384

_PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
HOST_LIBRARY_PATH = os.path.join(_PACKAGE_DIR, "libentropack_host.so")
_host = None


def host_library() -> ctypes.CDLL:
    global _host
    if _host is None:
        if not os.path.exists(HOST_LIBRARY_PATH):
            raise ImportError(f"{HOST_LIBRARY_PATH} is missing: build it with `python -m entropack_amd.build`")
        lib = ctypes.CDLL(HOST_LIBRARY_PATH)
        p, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        lib.hc_quantize.argtypes = [p, p, i64, ctypes.c_float, p, i64, p, p, i32]
        lib.hc_quantize.restype = None
        lib.hc_levels.argtypes = [p, p, i64, p, i32]
        lib.hc_levels.restype = None
        lib.hc_stream_stats.argtypes = [p, p, i64, p]
        lib.hc_stream_stats.restype = None
        lib.hc_stream_counts.argtypes = [p, p, i64, p, p, p]
        lib.hc_stream_counts.restype = None
        lib.hc_normalize_counts.argtypes = [p, i64, i64, p]
        lib.hc_normalize_counts.restype = i32
        lib.hc_normalize_streams.argtypes = [p, p, i64, i64, p]
        lib.hc_normalize_streams.restype = i32
        lib.hc_tile_ans_normalize_counts.argtypes = [p, i64, i64, p]
        lib.hc_tile_ans_normalize_counts.restype = i32
        lib.hc_rans_encode.argtypes = [p, p, i64, p, p, p, p, i32, i32, p, p, ctypes.POINTER(ctypes.c_void_p), i32]
        lib.hc_rans_encode.restype = i32
        lib.hc_tile_ans_encode.argtypes = [p, i64, i32, i64, i32, p, p, p, p, p, ctypes.POINTER(ctypes.c_void_p), i32]
        lib.hc_tile_ans_encode.restype = i32
        lib.hc_free.argtypes = [p]
        lib.hc_free.restype = None
        _host = lib
    return _host


def _threads() -> int:
    return max(1, min(torch.get_num_threads(), os.cpu_count() or 1))


def _address(array: np.ndarray) -> int:
    return array.ctypes.data


# ---- quantisation ----------------------------------------------------------------------------------------------

class Quantized:
    """Coset bit and the eight integer fields (z0..z6, m) of every vector, as the C kernels hold them."""

    def __init__(self, coset: np.ndarray, fields: np.ndarray):
        self.coset, self.fields = coset, fields          # int8[V], int32[V, 8]

    @property
    def vectors(self) -> int:
        return int(self.coset.size)

    def stats(self) -> np.ndarray:
        """int64[17, 3]: n, min, max of each stream."""
        out = np.zeros((NUM_STREAMS, 3), dtype=np.int64)
        host_library().hc_stream_stats(_address(self.coset), _address(self.fields), self.vectors, _address(out))
        out[0, 1] = 0                    # the coset stream always counts from symbol 0
        return out

    def histograms(self, stats: np.ndarray):
        """Per stream: counts over value - min (empty array for an empty stream)."""
        alphabets = np.where(stats[:, 0] > 0, stats[:, 2] - stats[:, 1] + 1, 0)
        starts = np.concatenate([[0], np.cumsum(alphabets)]).astype(np.int64)
        counts = np.zeros(int(starts[-1]), dtype=np.int64)
        minima = np.ascontiguousarray(stats[:, 1])
        host_library().hc_stream_counts(_address(self.coset), _address(self.fields), self.vectors, _address(minima),
                                        _address(starts), _address(counts))
        return [counts[starts[s]:starts[s + 1]] for s in range(NUM_STREAMS)]

    def levels(self) -> torch.Tensor:
        out = np.empty((self.vectors, LATTICE_DIM), dtype=np.float32)
        host_library().hc_levels(_address(self.coset), _address(self.fields), self.vectors, _address(out), _threads())
        return torch.from_numpy(out)

    def planes(self):
        """(coset int8 [V], fields int32 [V, 8]) as torch tensors over the same memory."""
        return torch.from_numpy(self.coset), torch.from_numpy(self.fields)


def quantize(x: np.ndarray, rms: np.ndarray, scale: float, rows_selected: np.ndarray | None = None) -> Quantized:
    rows, cols = x.shape
    picked = rows if rows_selected is None else int(rows_selected.size)
    vectors = picked * (cols // LATTICE_DIM)
    coset = np.empty(vectors, dtype=np.int8)
    fields = np.empty((vectors, NUM_FIELDS), dtype=np.int32)
    host_library().hc_quantize(
        _address(x), _address(rms), cols, ctypes.c_float(scale), None if rows_selected is None else _address(rows_selected),
        picked, _address(coset), _address(fields), _threads())
    return Quantized(coset, fields)


class HostQuantizer:
    """The float32 matrix and its row RMS on the CPU; quantises and refits through libentropack_host.so.

    The scale search below talks to this interface only (`rows`, `cols`, `all_zero`, `quantize`, `refit`), which the
    device lane implements with its own kernels.
    """

    def __init__(self, x_t: torch.Tensor, rms_t: torch.Tensor):
        self.x_t, self.rms_t = x_t, rms_t
        self.rows, self.cols = x_t.shape
        self._x = x_t.numpy()
        self._rms = np.ascontiguousarray(rms_t.squeeze(1).numpy())

    def all_zero(self) -> bool:
        return float(self.x_t.abs().amax()) == 0.0

    def quantize(self, scale: float, rows_selected: np.ndarray | None = None) -> Quantized:
        return quantize(self._x, self._rms, scale, rows_selected)

    def refit(self, q: Quantized, scale: float) -> torch.Tensor:
        return refit_row_scales(self.x_t, self.rms_t, q, scale)[0]

    def refit_with_error(self, q: Quantized, scale: float):
        """(row scales, squared error of every row at its fitted scale)."""
        return refit_row_scales(self.x_t, self.rms_t, q, scale)

    def assemble(self, coset: torch.Tensor, fields: torch.Tensor) -> Quantized:
        """Quantised vectors from integer tensors [V] and [V, 8] (rows picked from several quantisations)."""
        return Quantized(np.ascontiguousarray(coset.numpy().astype(np.int8)), np.ascontiguousarray(fields.numpy().astype(np.int32)))


# ---- frequency tables and the size model -------------------------------------------------------------------------

def normalize_counts(counts: np.ndarray, table_size: int) -> np.ndarray:
    """Largest-remainder (Hamilton) allocation of `table_size` slots, every present symbol getting at least one.

    A surplus is handed out by descending residual, a deficit taken back by ascending residual from symbols still
    above 1; ties go to the smaller symbol, and a symbol can be visited again in a later pass. The arithmetic is
    hc_normalize_counts of libentropack_host.so (float64 shares, as the reference's numpy code computes them).
    """
    counts = np.ascontiguousarray(counts, dtype=np.int64)
    if counts.size == 0 or int(counts.sum()) == 0:
        raise ValueError("cannot build an rANS table from an empty symbol stream")
    if counts.size > table_size:
        raise ValueError(
            f"E8 coordinate alphabet {counts.size} exceeds rANS table_size {table_size}; "
            "raise prob_bits or coarsen the lattice scale")
    freq = np.empty(counts.size, dtype=np.uint16)
    status = host_library().hc_normalize_counts(_address(counts), counts.size, table_size, _address(freq))
    if status == -3:
        raise MemoryError("frequency normalisation ran out of memory")
    if status != 0:
        raise ValueError("unable to normalize rANS frequencies")
    return freq


def modelled_bytes(histograms, sizes, rows: int, prob_bits: int, tile_elements: int) -> float:
    """Analytic container size for a set of stream histograms (reference rans.py:224-258 + eager.py:102-107).

    Per coded stream the reference adds count * (prob_bits - log2(freq)) over the symbols present, in float64 with
    numpy's sum, and the streams' sums in stream order. The same numbers come out of one normalisation call and one
    pass of element-wise arithmetic over the histograms laid end to end, with numpy's sum over each stream's slice
    (element-wise results and a slice's sum do not depend on where in an array the elements lie).
    """
    table_size = 1 << prob_bits
    coded = [hist for n, hist in zip(sizes, histograms) if n and hist.size <= table_size]
    overflow_bits = float(sum(n * prob_bits for n, hist in zip(sizes, histograms) if not (n and hist.size <= table_size)))
    bits = 0.0
    table_bytes = 0
    if coded:
        counts = np.ascontiguousarray(np.concatenate(coded), dtype=np.int64)
        starts = np.zeros(len(coded) + 1, dtype=np.int64)
        np.cumsum([hist.size for hist in coded], out=starts[1:])
        freq = np.empty(counts.size, dtype=np.uint16)
        status = host_library().hc_normalize_streams(_address(counts), _address(starts), len(coded), table_size, _address(freq))
        if status == -3:
            raise MemoryError("frequency normalisation ran out of memory")
        if status != 0:
            raise ValueError("unable to normalize rANS frequencies")
        live = counts > 0
        terms = counts[live].astype(np.float64) * (prob_bits - np.log2(freq[live].astype(np.float64)))
        ends = np.concatenate([[0], np.cumsum(live)])[starts]          # where each stream's present symbols begin in `terms`
        for k in range(len(coded)):
            bits += float(np.sum(terms[ends[k]:ends[k + 1]]))
        table_bytes = 2 * counts.size
    tile_vectors = vector_tile_elements(tile_elements)
    tiles = max(1, (sizes[0] + tile_vectors - 1) // tile_vectors)
    payload_words = int(np.ceil(max(0.0, bits - tiles * NUM_STATES * 16) / 16.0))
    coded_bytes = payload_words * 2 + tiles * NUM_STATES * 4 + (tiles + 1) * 4 + table_bytes
    return coded_bytes + overflow_bits / 8 + rows * 4 + MODEL_LAYOUT_BYTES + MODEL_STREAM_META_BYTES + MODEL_SLACK_BYTES


def _model_of(q, rows: int, prob_bits: int, tile_elements: int) -> float:
    stats = q.stats()
    return modelled_bytes(q.histograms(stats), [int(n) for n in stats[:, 0]], rows, prob_bits, tile_elements)


def _largest_alphabet(q) -> int:
    stats = q.stats()
    spans = np.where(stats[:, 0] > 0, stats[:, 2] - stats[:, 1] + 1, 0)
    return int(spans.max())


def bisect_scale(quantizer, target_bpp, prob_bits, tile_elements, iterations, max_vectors) -> float:
    """Geometric bisection of the lattice scale on [0.001, 8] against the size model, on a seeded row subsample."""
    rows, cols = quantizer.rows, quantizer.cols
    per_row = cols // LATTICE_DIM
    sample_rows = max(1, min(rows, max_vectors // per_row))
    picked = None
    if sample_rows < rows:
        generator = torch.Generator().manual_seed(rows * SUBSAMPLE_SEED_MULTIPLIER + cols)
        picked = np.ascontiguousarray(torch.randperm(rows, generator=generator)[:sample_rows].numpy(), dtype=np.int64)
    elements = sample_rows * cols
    low, high = 0.001, 8.0
    for _ in range(iterations):
        middle = math.sqrt(low * high)
        size = _model_of(quantizer.quantize(middle, picked), sample_rows, prob_bits, tile_elements)
        if 8 * size / elements > target_bpp:
            low = middle
        else:
            high = middle
    return math.sqrt(low * high)


def refit_row_scales(x_t: torch.Tensor, rms_t: torch.Tensor, q: Quantized, scale: float):
    """Least-squares scale of each row against the points chosen for it, and the squared error that scale leaves
    (float32 row sums, as torch computes them; the reference's eager.py:209-225)."""
    rows, cols = x_t.shape
    levels = q.levels().reshape(rows, cols)
    numerator = (x_t * levels).sum(1)
    denominator = levels.square().sum(1)
    scales = torch.where(denominator > 0, (numerator / denominator).clamp_min(MIN_RMS), scale * rms_t.squeeze(1))
    energy = x_t.square().sum(1)
    row_sse = torch.where(denominator > 0, (energy - numerator * numerator / denominator).clamp_min(0.0), energy)
    return scales, row_sse


def resolve_scale(quantizer, target_bpp, prob_bits, tile_elements, iterations, max_vectors, rdo_iterations=0, rdo_candidates=5):
    """Scale search plus the alphabet guard: grow an automatic prob_bits (to 15 at most) while an alphabet overflows
    the table, after that coarsen the scale by the overflow. With `rdo_iterations` > 0 the rows are then refined one by
    one (rdo.py), which can widen an alphabet again, so the guard looks at what that pass returns. Returns (quantised
    vectors, row scales, prob_bits)."""
    from . import rdo
    prob_bits, automatic = resolve_prob_bits(prob_bits, target_bpp)
    if quantizer.all_zero():
        q = quantizer.quantize(1.0)
        return q, quantizer.refit(q, 1.0), prob_bits
    clamped = False
    while True:
        table_size = 1 << prob_bits
        scale = bisect_scale(quantizer, target_bpp, prob_bits, tile_elements, iterations, max_vectors)
        grow = False
        while True:
            q = quantizer.quantize(scale)
            widest = _largest_alphabet(q)
            scales = None
            if widest <= table_size and rdo_iterations > 0:
                baseline = rdo.RowCandidate(q, *quantizer.refit_with_error(q, scale))
                rows = quantizer.rows
                q, scales = rdo.refine_rows(
                    quantizer, baseline, scale, rdo_iterations, rdo_candidates,
                    lambda stats, histograms: modelled_bytes(histograms, [int(n) for n in stats[:, 0]], rows, prob_bits, tile_elements))
                widest = _largest_alphabet(q)
            if widest <= table_size:
                break
            if automatic and prob_bits < 15:
                prob_bits += 1
                grow = True
                break
            clamped = True
            scale *= widest / table_size * ALPHABET_COARSEN_MARGIN
        if grow:
            continue
        if clamped:
            log.debug("lattice_rans coarsened the lattice scale to %.6g so a coordinate alphabet of %d fits the "
                      "%d-entry rANS table; actual_bpp for this tensor will fall below target_bpp", scale, widest, table_size)
        return q, (quantizer.refit(q, scale) if scales is None else scales), prob_bits


# ---- stream encode ---------------------------------------------------------------------------------------------

def stream_tables(stats: np.ndarray, histograms, prob_bits: int):
    """stream_meta and the normalised frequencies / cumulative frequencies of all streams, concatenated in stream order
    (int64 numpy arrays; entropack/schemes/lattice_rans/cuda.py:481-517 is the reference's form of this step)."""
    table_size = 1 << prob_bits
    meta = np.zeros((NUM_STREAMS, META_WIDTH), dtype=np.int64)
    freq_parts, cdf_parts = [], []
    cursor = 0
    for stream, hist in enumerate(histograms):
        n = int(stats[stream, 0])
        meta[stream, META_N_SYMBOLS] = n
        meta[stream, META_SYM_MIN] = int(stats[stream, 1]) if n else 0
        meta[stream, META_FREQ_OFFSET] = cursor
        meta[stream, META_ALPHABET] = hist.size if n else 0
        if n:
            freq = normalize_counts(hist, table_size).astype(np.int64)
            freq_parts.append(freq)
            cdf_parts.append(np.concatenate([[0], np.cumsum(freq)[:-1]]))
            cursor += hist.size
    freq_all = np.concatenate(freq_parts) if freq_parts else np.zeros(0, dtype=np.int64)
    cdf_all = np.concatenate(cdf_parts) if cdf_parts else np.zeros(0, dtype=np.int64)
    return meta, freq_all, cdf_all


def encode_streams(q: Quantized, prob_bits: int, tile_elements: int):
    """Frequency tables + tiled rANS encode. Returns payload, states, offsets, stream_meta, freq_tables (numpy)."""
    stats = q.stats()
    meta, freq_all, cdf_all = stream_tables(stats, q.histograms(stats), prob_bits)

    tile_vectors = vector_tile_elements(tile_elements)
    tiles = max(1, (q.vectors + tile_vectors - 1) // tile_vectors)
    states = np.empty((tiles, NUM_STATES), dtype=np.uint32)
    offsets = np.zeros(tiles + 1, dtype=np.uint32)
    minima = np.ascontiguousarray(meta[:, META_SYM_MIN])
    starts = np.ascontiguousarray(meta[:, META_FREQ_OFFSET])
    freq32 = np.ascontiguousarray(freq_all.astype(np.uint32))
    cdf32 = np.ascontiguousarray(cdf_all.astype(np.uint32))
    handle = ctypes.c_void_p()
    status = host_library().hc_rans_encode(
        _address(q.coset), _address(q.fields), q.vectors, _address(minima), _address(starts), _address(freq32),
        _address(cdf32), prob_bits, tile_vectors, _address(states), _address(offsets), ctypes.byref(handle), _threads())
    if status != 0:
        raise MemoryError("rANS encode ran out of memory" if status == -1 else "payload exceeds 2**32 words")
    try:
        words = int(offsets[-1])
        payload = np.ctypeslib.as_array(ctypes.cast(handle, ctypes.POINTER(ctypes.c_uint16)), shape=(max(words, 1),))[:words].copy()
    finally:
        host_library().hc_free(handle)
    return payload, states, offsets, meta, freq_all.astype(np.uint16)


def _as_torch(array: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    """numpy unsigned arrays -> torch tensors of the matching unsigned dtype (via a same-width signed view)."""
    signed = {torch.uint16: np.int16, torch.uint32: np.int32}.get(dtype)
    if signed is None:
        return torch.from_numpy(np.ascontiguousarray(array))
    return torch.from_numpy(np.ascontiguousarray(array).view(signed)).view(dtype)


def check_encode_request(weight) -> None:
    if weight.shape[1] % LATTICE_DIM:
        raise ValueError(
            f"lattice_rans quantizes whole E8 vectors, so the column count must be a multiple of {LATTICE_DIM}; got cols={weight.shape[1]}")


def row_rms(x_t: torch.Tensor, source_dtype) -> torch.Tensor:
    """float32 [rows, 1]: root mean square of every row, at least MIN_RMS (torch's reductions on the tensor's device)."""
    rms_t = x_t.square().mean(dim=1, keepdim=True).sqrt().clamp_min(MIN_RMS)
    if not bool(torch.isfinite(rms_t).all()):
        raise ValueError(
            f"lattice_rans normalizes rows in fp32, and the row RMS of this {source_dtype} tensor overflowed; rescale the source")
    return rms_t


def encode(*, weight, target_bpp, prob_bits, tile_elements, row_rdo_iterations=0, row_rdo_candidates=5,
           scale_search_iterations=12, scale_search_max_vectors=262144) -> LatticeBuffers:
    check_encode_request(weight)
    device = weight.device
    x_t = weight.detach().to("cpu").float().contiguous()
    rows, cols = x_t.shape
    rms_t = row_rms(x_t, weight.dtype)
    q, scales, prob_bits = resolve_scale(
        HostQuantizer(x_t, rms_t), float(target_bpp), None if prob_bits in (None, 0) else int(prob_bits), int(tile_elements),
        int(scale_search_iterations), int(scale_search_max_vectors), int(row_rdo_iterations), int(row_rdo_candidates))
    payload, states, offsets, meta, freq_tables = encode_streams(q, prob_bits, int(tile_elements))
    return LatticeBuffers(
        payload=_as_torch(payload, torch.uint16).to(device), offsets=_as_torch(offsets, torch.uint32).to(device),
        states=_as_torch(states, torch.uint32).to(device), stream_meta=torch.from_numpy(meta.astype(np.int32)).to(device),
        freq_tables=_as_torch(freq_tables, torch.uint16).to(device), scales=scales.contiguous().to(device),
        layout=make_layout(cols, prob_bits, int(tile_elements)).to(device),
    )


def decode(buffers, *, shape, dtype, threads_per_block=None, l2_prefetch=True):
    raise RuntimeError(
        "this package has no CPU decoder: lattice_rans containers are decoded by the hip lane (MI355X). "
        "Pass execution_backend='hip' on a machine with a gfx950 device.")
