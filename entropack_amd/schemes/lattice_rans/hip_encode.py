"""Device encoder of the `hip` lane: `compress` for a weight that already sits on an MI355X.

The lane contract is the reference CUDA lane's (entropack/schemes/lattice_rans/cuda.py:561-597): a float matrix on the
device in, `LatticeBuffers` on the same device out. The orchestration is the CPU lane's (`eager.resolve_scale`: the
same seeded row subsample, geometric bisection against the same size model, alphabet guard, Hamilton-normalised
tables), driven through the quantizer interface with this module's kernels behind it, so the two lanes differ only
in the row RMS (torch's reduction on the device instead of on the CPU, and a correctly rounded root where the CPU's
vectorised one is not always) and in the order the refit adds its float32 row sums. From the same row RMS the lattice
scale, coset bits, fields, tables, states, offsets and payload are bit-identical to the CPU lane's.

Kernels: `ep_hip_encode_*` of libentropack_hip.so (csrc/ep_encode.hip). Nothing here runs on the CPU except the
table construction over the 17 histograms; a missing library or device raises.
"""
import numpy as np
import torch

from ...backends import hip as _hip
from . import eager
from .format import (
    META_FREQ_OFFSET, META_SYM_MIN, NUM_FIELDS, NUM_STATES, NUM_STREAMS, LatticeBuffers, make_layout, vector_tile_elements,
)

SUMMARY_WORDS = 33          # EP_HIP_ENCODE_SUMMARY_WORDS
SYMBOLS_PER_VECTOR = 9


def _stream(device: torch.device) -> int:
    return _hip.current_stream(device)


class DeviceQuantized:
    """Coset bits and fields of every vector on the device, with the summary the quantise kernel left."""

    def __init__(self, coset: torch.Tensor, fields: torch.Tensor, summary: np.ndarray):
        self.coset, self.fields = coset, fields          # int8[V], int32[V, 8]
        self._summary = summary                          # int64[33] on the host

    @property
    def vectors(self) -> int:
        return int(self.coset.numel())

    def stats(self) -> np.ndarray:
        """int64[17, 3]: n, min, max of each stream (zeros for an empty stream; the coset stream counts from 0)."""
        out = np.zeros((NUM_STREAMS, 3), dtype=np.int64)
        ones = int(self._summary[2 * (NUM_STREAMS - 1)])
        out[0] = (self.vectors, 0, 1 if ones else 0)
        for k in range(NUM_STREAMS - 1):
            n = ones if k & 1 else self.vectors - ones
            if n:
                out[1 + k] = (n, int(self._summary[2 * k]), int(self._summary[2 * k + 1]))
        return out

    def histograms(self, stats: np.ndarray):
        """Per stream: counts over value - min (empty array for an empty stream), as numpy int64."""
        alphabets = np.where(stats[:, 0] > 0, stats[:, 2] - stats[:, 1] + 1, 0)
        starts = np.concatenate([[0], np.cumsum(alphabets)]).astype(np.int64)
        total = int(starts[-1])
        if total >= 1 << 31:
            raise ValueError("lattice_rans alphabets are too wide to count on the device; coarsen the lattice scale")
        device = self.coset.device
        relative = torch.from_numpy((starts[:NUM_STREAMS] - stats[:, 1]).astype(np.int32)).to(device)
        bins = torch.empty(total, dtype=torch.int64, device=device)
        _hip.check("ep_hip_encode_histogram", _hip.library().ep_hip_encode_histogram(
            self.coset.data_ptr(), self.fields.data_ptr(), self.vectors, relative.data_ptr(), total, bins.data_ptr(), _stream(device)))
        counts = bins.cpu().numpy()
        if int(counts.sum()) != SYMBOLS_PER_VECTOR * self.vectors:
            raise RuntimeError("lattice_rans device histogram lost symbols: the stream minima do not cover the fields")
        return [counts[starts[s]:starts[s + 1]] for s in range(NUM_STREAMS)]

    def planes(self):
        """(coset int8 [V], fields int32 [V, 8]) on the device."""
        return self.coset, self.fields


class DeviceQuantizer:
    """`eager.HostQuantizer`'s interface over a float32 matrix and its row RMS on the device."""

    def __init__(self, x: torch.Tensor, rms: torch.Tensor):
        if x.dtype != torch.float32 or not x.is_contiguous() or x.device.type != "cuda":
            raise ValueError("the device encoder takes a contiguous float32 matrix on the GPU")
        self.x, self.rms = x, rms.reshape(-1).contiguous()
        self.rows, self.cols = x.shape
        self._picked_host = None
        self._picked_device = None

    def all_zero(self) -> bool:
        return float(self.x.abs().amax()) == 0.0

    def _row_index(self, rows_selected: np.ndarray) -> torch.Tensor:
        if self._picked_host is not rows_selected:                        # the search passes one array through all its iterations
            self._picked_device = torch.from_numpy(np.ascontiguousarray(rows_selected, dtype=np.int64)).to(self.x.device)
            self._picked_host = rows_selected
        return self._picked_device

    def quantize(self, scale: float, rows_selected: np.ndarray | None = None) -> DeviceQuantized:
        device = self.x.device
        picked = self.rows if rows_selected is None else int(rows_selected.size)
        index = None if rows_selected is None else self._row_index(rows_selected)
        if index is not None and picked and (int(rows_selected.min()) < 0 or int(rows_selected.max()) >= self.rows):
            raise IndexError("row subsample outside the matrix")
        vectors = picked * (self.cols // 8)
        coset = torch.empty(vectors, dtype=torch.int8, device=device)
        fields = torch.empty((vectors, NUM_FIELDS), dtype=torch.int32, device=device)
        summary = torch.empty(SUMMARY_WORDS, dtype=torch.int64, device=device)
        _hip.check("ep_hip_encode_quantize", _hip.library().ep_hip_encode_quantize(
            self.x.data_ptr(), self.rms.data_ptr(), self.cols, float(scale), 0 if index is None else index.data_ptr(), picked,
            coset.data_ptr(), fields.data_ptr(), summary.data_ptr(), _stream(device)))
        return DeviceQuantized(coset, fields, summary.cpu().numpy())

    def _refit(self, q: DeviceQuantized, scale: float, with_error: bool):
        device = self.x.device
        scales = torch.empty(self.rows, dtype=torch.float32, device=device)
        row_sse = torch.empty(self.rows, dtype=torch.float32, device=device) if with_error else None
        _hip.check("ep_hip_encode_row_scales", _hip.library().ep_hip_encode_row_scales(
            self.x.data_ptr(), self.rms.data_ptr(), self.cols, float(scale), self.rows, q.coset.data_ptr(), q.fields.data_ptr(),
            scales.data_ptr(), row_sse.data_ptr() if with_error else 0, _stream(device)))
        return scales, row_sse

    def refit(self, q: DeviceQuantized, scale: float) -> torch.Tensor:
        return self._refit(q, scale, False)[0]

    def refit_with_error(self, q: DeviceQuantized, scale: float):
        """(row scales, squared error of every row at its fitted scale), float32 on the device."""
        return self._refit(q, scale, True)

    def assemble(self, coset: torch.Tensor, fields: torch.Tensor) -> DeviceQuantized:
        return quantized_from_planes(coset, fields)


def quantized_from_planes(coset: torch.Tensor, fields: torch.Tensor) -> DeviceQuantized:
    """Quantised vectors from integer tensors [V] and [V, 8] (rows picked from several quantisations); the summary the
    quantise kernel would have left is taken with torch reductions on the tensors' device."""
    coset = coset.to(torch.int8).contiguous()
    fields = fields.to(torch.int32).contiguous()
    summary = np.empty(SUMMARY_WORDS, dtype=np.int64)
    halves = coset.bool()
    for bit, mask in ((0, ~halves), (1, halves)):
        chosen = fields[mask]
        if chosen.shape[0]:
            low, high = chosen.amin(0).cpu().numpy(), chosen.amax(0).cpu().numpy()
        else:
            low = np.full(NUM_FIELDS, np.iinfo(np.int64).max, dtype=np.int64)
            high = np.full(NUM_FIELDS, np.iinfo(np.int64).min, dtype=np.int64)
        for field in range(NUM_FIELDS):
            summary[2 * (2 * field + bit)], summary[2 * (2 * field + bit) + 1] = int(low[field]), int(high[field])
    summary[2 * (NUM_STREAMS - 1)] = int(halves.sum())
    return DeviceQuantized(coset, fields, summary)


def table_entries(freq_all: np.ndarray, cdf_all: np.ndarray) -> torch.Tensor:
    """int64 per table position: frequency | cumulative frequency << 16 in the low half, the reciprocal the kernel divides
    with, min(floor(2^32 / frequency), 2^32 - 1), in the high half."""
    freq = freq_all.astype(np.uint64)
    reciprocal = np.minimum((np.uint64(1) << np.uint64(32)) // np.maximum(freq, np.uint64(1)), np.uint64(0xFFFFFFFF))
    packed = freq | (cdf_all.astype(np.uint64) << np.uint64(16)) | (reciprocal << np.uint64(32))
    return torch.from_numpy(packed.view(np.int64))


def encode_streams(q: DeviceQuantized, prob_bits: int, tile_elements: int):
    """Frequency tables (host, from the device histograms) and the tiled rANS encode (device). Returns payload
    uint16[words], states uint32[tiles, 32], offsets uint32[tiles + 1] on the device, and stream_meta / freq_tables as
    numpy arrays."""
    device = q.coset.device
    lib = _hip.library()
    stats = q.stats()
    meta, freq_all, cdf_all = eager.stream_tables(stats, q.histograms(stats), prob_bits)
    entries = table_entries(freq_all, cdf_all).to(device)
    relative = torch.from_numpy((meta[:, META_FREQ_OFFSET] - meta[:, META_SYM_MIN]).astype(np.int32)).to(device)

    tile_vectors = vector_tile_elements(tile_elements)
    tiles = max(1, (q.vectors + tile_vectors - 1) // tile_vectors)
    states = torch.empty((tiles, NUM_STATES), dtype=torch.int32, device=device)
    tile_words = torch.empty(tiles, dtype=torch.int32, device=device)
    scratch = torch.empty(tiles * tile_vectors * SYMBOLS_PER_VECTOR, dtype=torch.int16, device=device)
    error = torch.zeros(1, dtype=torch.int32, device=device)
    offsets = torch.empty(tiles + 1, dtype=torch.int32, device=device)
    total = torch.empty(1, dtype=torch.int64, device=device)
    _hip.check("ep_hip_encode_rans", lib.ep_hip_encode_rans(
        q.coset.data_ptr(), q.fields.data_ptr(), q.vectors, entries.data_ptr(), relative.data_ptr(), int(entries.numel()), prob_bits,
        tile_vectors, states.data_ptr(), tile_words.data_ptr(), scratch.data_ptr(), error.data_ptr(), _stream(device)))
    _hip.check("ep_hip_encode_offsets", lib.ep_hip_encode_offsets(
        tile_words.data_ptr(), tiles, offsets.data_ptr(), total.data_ptr(), _stream(device)))
    words = int(total.item())
    if int(error.item()):
        raise RuntimeError("lattice_rans device encode met a symbol outside its frequency tables")
    if words >= 1 << 32:
        raise ValueError("lattice_rans payload exceeds uint32 offset capacity")
    payload = torch.empty(words, dtype=torch.int16, device=device)
    if words:
        _hip.check("ep_hip_encode_gather", lib.ep_hip_encode_gather(
            scratch.data_ptr(), offsets.data_ptr(), tiles, tile_vectors * SYMBOLS_PER_VECTOR, payload.data_ptr(), _stream(device)))
    return payload.view(torch.uint16), states.view(torch.uint32), offsets.view(torch.uint32), meta, freq_all.astype(np.uint16)


def encode_normalised(x: torch.Tensor, rms: torch.Tensor, *, target_bpp, prob_bits, tile_elements, scale_search_iterations=12,
                      scale_search_max_vectors=262144, row_rdo_iterations=0, row_rdo_candidates=5) -> LatticeBuffers:
    """The container of the float32 device matrix `x` whose rows are normalised by `rms` (float32 [rows, 1], on the device).
    With the CPU lane's row RMS this is the CPU lane's container except for the order of the refit's float32 sums."""
    device = x.device
    cols = x.shape[1]
    q, scales, prob_bits = eager.resolve_scale(
        DeviceQuantizer(x, rms), float(target_bpp), None if prob_bits in (None, 0) else int(prob_bits), int(tile_elements),
        int(scale_search_iterations), int(scale_search_max_vectors), int(row_rdo_iterations), int(row_rdo_candidates))
    payload, states, offsets, meta, freq_tables = encode_streams(q, prob_bits, int(tile_elements))
    return LatticeBuffers(
        payload=payload, offsets=offsets, states=states, stream_meta=torch.from_numpy(meta.astype(np.int32)).to(device),
        freq_tables=eager._as_torch(freq_tables, torch.uint16).to(device), scales=scales.contiguous(),
        layout=make_layout(cols, prob_bits, int(tile_elements)).to(device),
    )


def row_rms(x: torch.Tensor, source_dtype) -> torch.Tensor:
    """float32 [rows, 1]: root of the float32 mean of squares of every row, at least eager.MIN_RMS. The root is taken in
    float64 and rounded once, which is the correctly rounded float32 root (torch's float32 root on the device is not)."""
    rms = x.square().mean(dim=1, keepdim=True).double().sqrt().float().clamp_min(eager.MIN_RMS)
    if not bool(torch.isfinite(rms).all()):
        raise ValueError(
            f"lattice_rans normalizes rows in fp32, and the row RMS of this {source_dtype} tensor overflowed; rescale the source")
    return rms


def encode(*, weight, target_bpp, prob_bits, tile_elements, row_rdo_iterations=0, row_rdo_candidates=5,
           scale_search_iterations=12, scale_search_max_vectors=262144) -> LatticeBuffers:
    eager.check_encode_request(weight)
    if weight.device.type != "cuda":
        raise ValueError("the hip lane encodes tensors that are on the GPU; use execution_backend='eager' for CPU tensors")
    x = weight.detach().float().contiguous()
    return encode_normalised(x, row_rms(x, weight.dtype), target_bpp=target_bpp, prob_bits=prob_bits, tile_elements=tile_elements,
                             scale_search_iterations=scale_search_iterations, scale_search_max_vectors=scale_search_max_vectors,
                             row_rdo_iterations=row_rdo_iterations, row_rdo_candidates=row_rdo_candidates)
