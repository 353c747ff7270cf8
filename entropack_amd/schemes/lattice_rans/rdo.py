"""Optional per-row rate-distortion refinement of a lattice_rans encode (`row_rdo_iterations > 0`).

After the scale search has fixed one lattice scale for the tensor, every row may instead take the points of a slightly
finer or coarser scale (a short ladder of ratios around 1), chosen so that the squared error falls while the modelled
size of the container stays at what the single scale would have cost. Restates the reference's pass
(entropack/schemes/lattice_rans/rdo.py:12-162 and eager.py:229-252) with the same tensor operations in the same order,
so that on the CPU lane the choice of every row, and with it the container, is the reference's bit for bit (golden
fixtures `rdo*`). The module is written against the quantizer interface of eager.py and torch tensors on whatever device
the quantizer computes on, so the device lane runs the same pass with its own kernels behind it.
"""
import numpy as np
import torch

from .format import NUM_FIELDS, NUM_STREAMS

RATIO_LOW, RATIO_HIGH = 0.70, 1.45
SMOOTHING = 0.5                 # added to every count when a symbol is priced: unseen symbols stay affordable
GROWTH_STEPS, BISECTION_STEPS = 50, 20


def scale_ratios(count: int) -> tuple:
    """1.0 first, then one geometric midpoint of the (relatively) widest gap between RATIO_LOW, the points so far and
    RATIO_HIGH per further point; the first of equally wide gaps."""
    points = [1.0]
    while len(points) < count:
        fence = [RATIO_LOW, *points, RATIO_HIGH]
        widest = max(range(1, len(fence)), key=lambda j: fence[j] / fence[j - 1])
        points.insert(widest - 1, (fence[widest] * fence[widest - 1]) ** 0.5)
    return tuple(points)


class RowCandidate:
    """The whole tensor quantised at one scale of the ladder: its vectors, statistics, refitted scales, squared errors."""

    def __init__(self, quantized, scales: torch.Tensor, row_sse: torch.Tensor):
        self.quantized, self.scales, self.row_sse = quantized, scales, row_sse
        self.stats = quantized.stats()
        self.coset, self.fields = quantized.planes()            # [V], [V, 8] integer tensors


def _stream_spans(candidates):
    """Per stream, the least and greatest value any candidate holds (0, 0 for a stream empty everywhere)."""
    lows, highs = [0] * NUM_STREAMS, [0] * NUM_STREAMS
    for stream in range(NUM_STREAMS):
        spans = [(int(c.stats[stream, 1]), int(c.stats[stream, 2])) for c in candidates if c.stats[stream, 0] > 0]
        if spans:
            lows[stream] = min(low for low, _ in spans)
            highs[stream] = max(high for _, high in spans)
    return lows, highs


class PriceList:
    """-log2 of the smoothed relative frequency of every value of every stream, over the joint spans, as one float32
    tensor with the start of each stream and its least value beside it (int32, like the indices built from them)."""

    def __init__(self, stats: np.ndarray, histograms, lows, highs, device):
        parts, starts = [], [0]
        for stream, counts in enumerate(histograms):
            width = highs[stream] - lows[stream] + 1
            spread = np.zeros(width, dtype=np.float64)
            if counts.size:
                first = int(stats[stream, 1]) - lows[stream]
                spread[first:first + counts.size] = counts
            share = (spread + SMOOTHING) / (int(stats[stream, 0]) + SMOOTHING * width)
            parts.append(-np.log2(share).astype(np.float32))
            starts.append(starts[-1] + width)
        self.values = torch.from_numpy(np.concatenate(parts)).to(device)
        self.starts = torch.tensor(starts, dtype=torch.int32, device=device)
        self.lows = torch.tensor(lows, dtype=torch.int32, device=device)


def row_prices(rows: int, cols: int, candidate: RowCandidate, prices: PriceList) -> torch.Tensor:
    """float32 [rows]: the price of every row of a candidate; per vector the coset bit first, then fields 0 to 7, each
    added to the running float32 sum in that order, then torch's sum over the vectors of a row."""
    per_row = cols // NUM_FIELDS
    planes = candidate.fields.reshape(-1, NUM_FIELDS).t().contiguous().to(torch.int32)
    coset = candidate.coset.to(torch.int32)
    price = prices.values[prices.starts[0] + coset]
    for field in range(NUM_FIELDS):
        stream = 1 + 2 * field + coset
        price = price + prices.values[prices.starts[stream] + (planes[field] - prices.lows[stream])]
    return price.reshape(rows, per_row).sum(1)


def take_rows(rows: int, cols: int, candidates, choice: torch.Tensor):
    """coset int32 [V], fields int32 [V, 8] and scales [rows] with every row taken from the candidate `choice` names."""
    per_row = cols // NUM_FIELDS
    device = candidates[0].fields.device
    fields = torch.empty((rows, per_row, NUM_FIELDS), dtype=torch.int32, device=device)
    coset = torch.empty((rows, per_row), dtype=torch.int32, device=device)
    for index, candidate in enumerate(candidates):
        picked = torch.nonzero(choice == index, as_tuple=False).flatten()
        if picked.numel():
            fields[picked] = candidate.fields.reshape(rows, per_row, NUM_FIELDS)[picked].to(torch.int32)
            coset[picked] = candidate.coset.reshape(rows, per_row)[picked].to(torch.int32)
    scales = torch.stack([candidate.scales for candidate in candidates], dim=1)
    return coset.reshape(-1), fields.reshape(-1, NUM_FIELDS), scales[torch.arange(rows, device=choice.device), choice]


def cheapest_within(distortion: torch.Tensor, prices: torch.Tensor, every_row: torch.Tensor, budget) -> torch.Tensor:
    """Per row the candidate minimising distortion + lambda * price, for the smallest lambda found (doubling from a
    small start, then 20 geometric bisection steps) whose total price fits the budget; lambda = 0 when that fits."""
    greedy = distortion.argmin(1)
    if prices[every_row, greedy].sum() <= budget:
        return greedy
    choice = greedy
    low = 0.0
    high = max(float(distortion.mean().item()) * 1.0e-4, 1.0e-12)
    for _ in range(GROWTH_STEPS):
        trial = (distortion + high * prices).argmin(1)
        if prices[every_row, trial].sum() <= budget:
            break
        high *= 2.0
    for _ in range(BISECTION_STEPS):
        middle = high * 0.5 if low == 0.0 else (low * high) ** 0.5
        trial = (distortion + middle * prices).argmin(1)
        if prices[every_row, trial].sum() > budget:
            low = middle
        else:
            high = middle
            choice = trial
    return choice


def refine_rows(quantizer, baseline: RowCandidate, scale: float, iterations: int, candidate_count: int, size_model):
    """Runs the pass. `size_model(stats, histograms)` is the analytic container size in bytes. Returns the quantised
    vectors with every row from its chosen candidate, and the matching row scales."""
    rows, cols = quantizer.rows, quantizer.cols
    ratios = scale_ratios(candidate_count)
    home = ratios.index(1.0)
    candidates = []
    for index, ratio in enumerate(ratios):
        if index == home:
            candidates.append(baseline)
        else:
            quantized = quantizer.quantize(scale * ratio)
            candidates.append(RowCandidate(quantized, *quantizer.refit_with_error(quantized, scale * ratio)))
    device = baseline.fields.device
    lows, highs = _stream_spans(candidates)
    distortion = torch.stack([candidate.row_sse for candidate in candidates], dim=1)
    every_row = torch.arange(rows, device=device)
    choice = torch.full((rows,), home, dtype=torch.int64, device=device)
    coset, fields, scales = take_rows(rows, cols, candidates, choice)
    current = quantizer.assemble(coset, fields)
    allowance = size_model(baseline.stats, baseline.quantized.histograms(baseline.stats))
    for _ in range(iterations):
        stats = current.stats()
        histograms = current.histograms(stats)
        prices = PriceList(stats, histograms, lows, highs, device)
        price = torch.stack([row_prices(rows, cols, candidate, prices) for candidate in candidates], dim=1)
        budget = price[every_row, choice].sum() + 8 * (allowance - size_model(stats, histograms))
        choice = cheapest_within(distortion, price, every_row, budget)
        coset, fields, scales = take_rows(rows, cols, candidates, choice)
        current = quantizer.assemble(coset, fields)
    return current, scales
