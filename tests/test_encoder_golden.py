"""The package's CPU encoder against the containers the reference encoder wrote: same input + config -> same bytes."""
import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.schemes.lattice_rans import eager
from conftest import Golden

_DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32, "int8": torch.int8}


def _weight(golden):
    dtype = _DTYPES[golden.dtype]
    bits = torch.from_numpy(golden.weight_bits.copy())
    return bits.view(torch.int8) if dtype == torch.int8 else bits.view(dtype)


def test_compress_reproduces_the_reference_container(golden):
    container = ep.compress(_weight(golden), ep.EntroPackLossyConfig(execution_backend="eager", **golden.config_kwargs))
    assert container.compress_method == "lattice_rans"
    assert torch.equal(container.entropack_quant_state, torch.from_numpy(golden.quant_state))
    assert container.actual_bpp == golden.actual_bpp


def test_config_1_rate_and_error_window():
    """Benchmark configuration 1: 256x256 bf16 N(0, 0.02), seed 0, 3.5 bpp -> actual_bpp in [3.5, 3.6], rel-L2 near the
    E8 high-rate closed form 1.1065 * 2**-R for the payload rate R (container overhead excluded)."""
    golden = Golden("c1_256x256_bf16_3p5")
    torch.manual_seed(0)
    weight = (torch.randn(256, 256) * 0.02).to(torch.bfloat16)
    assert np.array_equal(weight.view(torch.int16).numpy(), golden.weight_bits)
    assert 3.5 <= golden.actual_bpp <= 3.6
    restored = torch.from_numpy(golden.restored_bits.copy()).view(torch.bfloat16).float()
    rel = ((restored - weight.float()).norm() / weight.float().norm()).item()
    payload_rate = 8 * 2 * golden.buffers["payload"].size / weight.numel()
    assert 0.9 * 1.1065 * 2 ** -payload_rate < rel < 1.35 * 1.1065 * 2 ** -payload_rate
    assert 0.11 < rel < 0.14


def hamilton_in_numpy(counts: np.ndarray, table_size: int) -> np.ndarray:
    """The allocation written out with numpy, step for step as the reference's rans.py:12-71 computes it (float64
    shares, floor, at least one slot per present symbol, stable sorts of the residuals, repeated passes): what the C
    routine behind `eager.normalize_counts` has to reproduce for every histogram, beyond the golden containers."""
    counts = np.asarray(counts, dtype=np.int64)
    seen = np.flatnonzero(counts)
    ideal = counts.astype(np.float64) * (table_size / int(counts.sum()))
    freq = np.floor(ideal).astype(np.int64)
    freq[seen] = np.maximum(freq[seen], 1)
    gap = table_size - int(freq.sum())
    if gap > 0:
        order = seen[np.argsort(-(ideal - freq)[seen], kind="stable")]
        while gap > 0:
            chosen = order[:gap]
            freq[chosen] += 1
            gap -= chosen.size
    elif gap < 0:
        rest = ideal - freq
        pool = seen[freq[seen] > 1]
        if pool.size == 0:
            raise ValueError("unable to normalize rANS frequencies")
        order = pool[np.argsort(rest[pool], kind="stable")]
        while gap < 0:
            alive = order[freq[order] > 1]
            if alive.size == 0:
                raise ValueError("unable to normalize rANS frequencies")
            chosen = alive[:-gap]
            freq[chosen] -= 1
            gap += chosen.size
    return freq.astype(np.uint16)


def test_hamilton_normalisation_matches_the_numpy_formulation():
    rng = np.random.default_rng(7)
    shortfalls = surpluses = 0
    for trial in range(3000):
        size = 1 << int(rng.integers(9, 16))
        width = int(rng.integers(1, min(size, 700) + 1))
        kind = trial % 5
        if kind == 0:
            counts = rng.integers(0, 50, size=width)
        elif kind == 1:                                   # a few heavy symbols over a long tail of ones: slots must be taken back
            counts = np.ones(width, dtype=np.int64)
            counts[rng.integers(0, width, size=3)] = rng.integers(10 ** 3, 10 ** 7, size=3)
        elif kind == 2:                                   # many exact ties
            counts = np.full(width, int(rng.integers(1, 9)), dtype=np.int64)
            counts[rng.integers(0, width, size=width // 3)] *= 2
        elif kind == 3:
            counts = np.floor(rng.exponential(40.0, size=width)).astype(np.int64)
        else:
            counts = (rng.integers(0, 2, size=width) * rng.integers(1, 10 ** 9, size=width)).astype(np.int64)
        if int(counts.sum()) == 0:
            counts[0] = 1
        try:
            want = hamilton_in_numpy(counts, size)
        except ValueError:
            with pytest.raises(ValueError):
                eager.normalize_counts(counts, size)
            continue
        floor_sum = int(np.maximum(np.floor(counts * (size / counts.sum())), counts > 0).sum())
        shortfalls += floor_sum < size
        surpluses += floor_sum > size
        got = eager.normalize_counts(counts, size)
        assert np.array_equal(got, want), (trial, counts.tolist(), size)
    assert shortfalls > 500 and surpluses > 200           # both directions were exercised, not only the common one
    assert eager.normalize_counts(np.array([5]), 2048).tolist() == [2048]
    full = eager.normalize_counts(np.ones(512, dtype=np.int64), 512)
    assert full.tolist() == [1] * 512
    with pytest.raises(ValueError):                      # every symbol already at one slot and still too many
        eager.normalize_counts(np.ones(513, dtype=np.int64), 512)


def size_model_stream_by_stream(histograms, sizes, rows, prob_bits, tile_elements):
    """The size model with one normalisation, one log2 and one sum per stream, as the reference's rans.py:224-258 and
    eager.py:102-107 go about it: what `eager.modelled_bytes`, which works on the histograms laid end to end, has to
    return to the last bit (the scale search compares its result with the target)."""
    from entropack_amd.schemes.lattice_rans.format import NUM_STATES, vector_tile_elements
    table_size = 1 << prob_bits
    bits, table_bytes, overflow_bits = 0.0, 0, 0.0
    for n, hist in zip(sizes, histograms):
        if n and hist.size <= table_size:
            freq = hamilton_in_numpy(hist, table_size)
            live = hist > 0
            bits += float(np.sum(hist[live].astype(np.float64) * (prob_bits - np.log2(freq[live].astype(np.float64)))))
            table_bytes += freq.size * 2
        else:
            overflow_bits += n * prob_bits
    tile_vectors = vector_tile_elements(tile_elements)
    tiles = max(1, (sizes[0] + tile_vectors - 1) // tile_vectors)
    payload_words = int(np.ceil(max(0.0, bits - tiles * NUM_STATES * 16) / 16.0))
    coded = payload_words * 2 + tiles * NUM_STATES * 4 + (tiles + 1) * 4 + table_bytes
    return (coded + overflow_bits / 8 + rows * 4 + eager.MODEL_LAYOUT_BYTES + eager.MODEL_STREAM_META_BYTES + eager.MODEL_SLACK_BYTES), bits


def test_size_model_matches_the_stream_by_stream_formulation():
    rng = np.random.default_rng(3)
    for trial in range(400):
        prob_bits = int(rng.integers(9, 16))
        histograms, sizes = [], []
        for stream in range(17):
            width = int(rng.integers(1, 90)) if rng.random() < 0.9 else int(rng.integers(400, 1200))      # some overflow a 9-bit table
            if stream and rng.random() < 0.1:
                histograms.append(np.zeros(0, dtype=np.int64)); sizes.append(0)                           # an empty stream
                continue
            hist = np.floor(rng.exponential(10.0 ** rng.uniform(0, 5), size=width)).astype(np.int64)
            hist[0] = max(hist[0], 1); hist[-1] = max(hist[-1], 1)
            histograms.append(hist); sizes.append(int(hist.sum()))
        want, want_bits = size_model_stream_by_stream(histograms, sizes, 64, prob_bits, 16384)
        assert eager.modelled_bytes(histograms, sizes, 64, prob_bits, 16384) == want, trial
        assert want_bits > 0.0


def test_hamilton_normalisation_properties():
    rng = np.random.default_rng(1)
    for size in (512, 2048):
        for _ in range(20):
            counts = rng.integers(0, 50, size=rng.integers(1, 60)).astype(np.int64)
            counts[rng.integers(0, counts.size)] += 1
            freq = eager.normalize_counts(counts, size).astype(np.int64)
            assert freq.sum() == size
            assert np.all((freq > 0) == (counts > 0))
    skew = np.array([1] * 600 + [10 ** 6], dtype=np.int64)                  # deficit path: 601 symbols into 512 slots fails
    with pytest.raises(ValueError):
        eager.normalize_counts(skew, 512)
    tight = np.array([1] * 500 + [10 ** 6], dtype=np.int64)
    freq = eager.normalize_counts(tight, 512)
    assert freq.sum() == 512 and freq[:500].tolist() == [1] * 500 and freq[500] == 12
    with pytest.raises(ValueError):
        eager.normalize_counts(np.zeros(4, dtype=np.int64), 512)


def test_encoder_rejects_what_the_reference_rejects():
    with pytest.raises(ValueError):
        ep.registry.get_scheme("lattice_rans").encode(torch.zeros(4, 4, 4), ep.EntroPackLossyConfig(execution_backend="eager"))
    with pytest.warns(ep.CompressionFallbackWarning):
        raw = ep.compress(torch.tensor([[float("inf")] * 8]), ep.EntroPackLossyConfig(execution_backend="eager"))
    assert raw.compress_method == "raw" and raw.header["requested"] == "lattice_rans"
    with pytest.raises(TypeError):
        ep.compress(raw, ep.EntroPackLossyConfig())


def test_row_refinement_lowers_the_error_at_the_same_size():
    """What the per-row pass is for: against the plain encode of the same weight at the same target, rows whose energy
    differs take different scales, the container does not grow and the squared error falls. (That the choice of every
    row is the reference's is what the `rdo*` fixtures check, byte for byte.)"""
    from entropack_amd.schemes.lattice_rans import rdo
    assert rdo.scale_ratios(1) == (1.0,)
    ladder = rdo.scale_ratios(5)
    assert len(ladder) == 5 and 1.0 in ladder and list(ladder) == sorted(ladder) and 0.70 < ladder[0] and ladder[-1] < 1.45
    assert set(rdo.scale_ratios(3)) <= set(ladder)
    golden = Golden("rdo2_rows_differ_128x128_bf16_2p5")
    weight = _weight(golden)
    plain = eager.encode(weight=weight, target_bpp=2.5, prob_bits=None, tile_elements=16384)
    refined = eager.encode(weight=weight, target_bpp=2.5, prob_bits=None, tile_elements=16384, row_rdo_iterations=2)
    assert not np.array_equal(refined.payload.view(torch.int16).numpy(), plain.payload.view(torch.int16).numpy())
    assert refined.payload.numel() <= plain.payload.numel() + 8
    restored = torch.from_numpy(golden.restored_bits.copy()).view(torch.bfloat16).float()
    quantizer = eager.HostQuantizer(weight.float().contiguous(), eager.row_rms(weight.float(), weight.dtype))
    q, scales, _ = eager.resolve_scale(quantizer, 2.5, None, 16384, 12, 262144)
    plain_dense = (q.levels().reshape(128, 128) * scales.unsqueeze(1)).to(torch.bfloat16).float()
    assert float((restored - weight.float()).square().sum()) < float((plain_dense - weight.float()).square().sum())
