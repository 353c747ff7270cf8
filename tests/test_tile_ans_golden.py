"""Lossless (`tile_ans`) containers, CPU side: the oracle and this package's encoder against the fixtures the reference
wrote (tests/golden/tile_ans), the container checks, and the encoder's own invariants."""
import os

import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.schemes.tile_ans import eager as tile_eager
from entropack_amd.schemes.tile_ans import format as tile_format
from conftest import GOLDEN_DIR
from oracle import c_oracle, tile_ans_oracle

TILE_DIR = os.path.join(GOLDEN_DIR, "tile_ans")
_UNSIGNED = {"payload": np.uint16, "offsets": np.uint32, "states": np.uint32, "decode_tables": np.uint32}
_TORCH = {"payload": torch.uint16, "offsets": torch.uint32, "states": torch.uint32, "decode_tables": torch.uint32}


def tile_names():
    with open(os.path.join(TILE_DIR, "INDEX.txt")) as handle:
        return [line.strip() for line in handle if line.strip()]


class TileGolden:
    """One reference-written lossless fixture."""

    def __init__(self, name):
        data = np.load(os.path.join(TILE_DIR, name + ".npz"), allow_pickle=False)
        self.name = name
        self.dtype = getattr(torch, str(data["dtype"]))
        self.shape = tuple(int(v) for v in data["shape"])
        self.options = {str(k): float(v) for k, v in zip(data["options_keys"], data["options_values"])}
        self.weight_bits = data["weight_bits"]
        self.quant_state = data["quant_state"]
        self.buffers = {}
        for key in tile_format.PACKED_KEYS:
            value = data["buf_" + key]
            self.buffers[key] = value.view(_UNSIGNED[key]) if key in _UNSIGNED else value

    @property
    def config(self):
        options = {k: (int(v) if k in ("tile_elements", "probability_bits") else v) for k, v in self.options.items()}
        return ep.TileANSConfig(execution_backend="eager", **options)

    @property
    def element_bytes(self):
        return torch.empty((), dtype=self.dtype).element_size()

    def tensor(self):
        if self.dtype == torch.bool:
            return torch.from_numpy(self.weight_bits.astype(bool)).reshape(self.shape)
        return torch.from_numpy(self.weight_bits.copy()).view(self.dtype).reshape(self.shape)

    def storage_bytes(self):
        return np.ascontiguousarray(self.weight_bits).reshape(-1).view(np.uint8)

    def torch_buffers(self):
        out = {}
        for key, value in self.buffers.items():
            if key in _TORCH:
                signed = value.view({2: np.int16, 4: np.int32}[value.dtype.itemsize])
                out[key] = torch.from_numpy(signed.copy()).view(_TORCH[key])
            else:
                out[key] = torch.from_numpy(value.copy())
        return out


@pytest.fixture(params=tile_names())
def tile_golden(request):
    return TileGolden(request.param)


def test_fixture_set_covers_the_format():
    goldens = [TileGolden(name) for name in tile_names()]
    modes = {tuple(int(m) for m in g.buffers["lane_modes"]) for g in goldens}
    assert {(1, 0), (1, 1), (0, 0), (0,), (1, 1, 1, 0)} <= modes and any(len(m) == 8 for m in modes)
    assert {int(g.buffers["layout"][1]) for g in goldens} == {9, 10, 11, 12}
    tails = {int(g.buffers["layout"][3]) % int(g.buffers["layout"][0]) % 32 for g in goldens}
    assert 0 in tails and len(tails) > 3                       # whole groups and several ragged tails
    escape = TileGolden("uint8_const_50x40_pb12").buffers["decode_tables"]
    assert np.all((escape >> 8) & 0xFFF == 0) and np.all(escape & 0xFF == 7)        # frequency 4096 is stored as 0


def test_oracles_reproduce_the_reference_bytes(tile_golden):
    literal = tile_ans_oracle.decode(tile_golden.buffers, tile_golden.element_bytes)
    fast = c_oracle.tile_ans_decode(tile_golden.buffers, tile_golden.element_bytes, threads=3)
    assert np.array_equal(literal, tile_golden.storage_bytes())
    assert np.array_equal(fast, tile_golden.storage_bytes())


def test_oracles_reject_damaged_streams():
    golden = TileGolden("int8_128x100_auto")
    short = dict(golden.buffers)
    short["offsets"] = golden.buffers["offsets"].copy()
    short["offsets"][1:] -= 1                                  # the first stream loses its last word
    with pytest.raises(ValueError, match="truncated|unread"):
        tile_ans_oracle.decode(short, 1)
    with pytest.raises(ValueError):
        c_oracle.tile_ans_decode(short, 1)
    derailed = dict(golden.buffers)
    derailed["states"] = golden.buffers["states"].copy()
    derailed["states"][0, 5] += 777
    try:                                                        # a wrong state either runs dry, leaves words, or decodes other bytes
        assert not np.array_equal(tile_ans_oracle.decode(derailed, 1), golden.storage_bytes())
    except ValueError:
        pass
    raw = TileGolden("int16_noise_60x50_auto")
    bad_raw = dict(raw.buffers)
    bad_raw["offsets"] = raw.buffers["offsets"].copy()
    bad_raw["offsets"][1] -= 1
    with pytest.raises(ValueError, match="raw lane"):
        tile_ans_oracle.decode(bad_raw, 2)
    with pytest.raises(ValueError, match="raw lane"):
        c_oracle.tile_ans_decode(bad_raw, 2)


def test_encoder_writes_the_reference_container_byte_for_byte(tile_golden):
    packed = ep.compress(tile_golden.tensor(), tile_golden.config)
    assert packed.compress_method == "tile_ans" and packed.dtype == tile_golden.dtype and tuple(packed.shape) == tile_golden.shape
    for key in tile_format.PACKED_KEYS:
        ours = packed.buffers[key]
        width = ours.element_size()
        got = ours.contiguous().view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[width]).numpy()
        want = tile_golden.buffers[key]
        want = want.view({1: np.uint8, 2: np.int16, 4: np.int32, 8: np.int64}[want.dtype.itemsize])
        assert got.shape == want.shape and np.array_equal(got, want), key
    assert np.array_equal(packed.entropack_quant_state.numpy(), tile_golden.quant_state)


def test_reference_blob_unpacks_and_validates(tile_golden):
    container = ep.CompressedTensor.unpack(torch.from_numpy(tile_golden.quant_state.copy()))
    assert container.compress_method == "tile_ans" and tuple(container.shape) == tile_golden.shape and container.dtype == tile_golden.dtype
    tile_format.validate_packed(container.buffers, tile_golden.shape, tile_golden.dtype)
    host = {key: (value.view({2: torch.int16, 4: torch.int32}[value.element_size()]).numpy().view(_UNSIGNED[key]) if key in _UNSIGNED else value.numpy())
            for key, value in container.buffers.items()}
    assert np.array_equal(c_oracle.tile_ans_decode(host, tile_golden.element_bytes), tile_golden.storage_bytes())


def test_validate_packed_catches_structural_damage():
    golden = TileGolden("f32_40x72_auto")
    good = golden.torch_buffers()
    tile_format.validate_packed(good, golden.shape, golden.dtype)
    with pytest.raises(ValueError, match="byte lanes"):
        tile_format.validate_packed(good, golden.shape, torch.bfloat16)
    with pytest.raises(ValueError, match="asks for"):
        tile_format.validate_packed(good, (40, 71), golden.dtype)
    for key in tile_format.PACKED_KEYS:
        with pytest.raises(ValueError, match="lacks buffers"):
            tile_format.validate_packed({k: v for k, v in good.items() if k != key}, golden.shape, golden.dtype)
    broken = dict(good, lane_modes=torch.tensor([1, 1, 2, 0], dtype=torch.uint8))
    with pytest.raises(ValueError, match="lane_modes must be"):
        tile_format.validate_packed(broken, golden.shape, golden.dtype)
    broken = dict(good, states=good["states"][:-1].clone()) if good["states"].shape[0] > 1 else dict(good, states=torch.zeros(3, 32, dtype=torch.uint32))
    with pytest.raises(ValueError, match="'states' must have shape"):
        tile_format.validate_packed(broken, golden.shape, golden.dtype)
    offsets = good["offsets"].clone()
    offsets.view(torch.int32)[1] -= 1
    with pytest.raises(ValueError, match="raw lane 0 does not hold"):
        tile_format.validate_packed(dict(good, offsets=offsets), golden.shape, golden.dtype)
    with pytest.raises(ValueError, match="int64\\[4\\]"):
        tile_format.validate_packed(dict(good, layout=good["layout"][:3].clone()), golden.shape, golden.dtype)


@pytest.mark.parametrize("seed", range(6))
def test_normalised_frequencies_keep_every_symbol_and_the_total(seed):
    rng = np.random.default_rng(seed)
    counts = np.zeros(256, dtype=np.int64)
    present = rng.choice(256, size=rng.integers(1, 256), replace=False)
    counts[present] = rng.integers(1, 10 ** rng.integers(1, 6), size=present.size)
    for bits in tile_format.SUPPORTED_PROB_BITS:
        if present.size > (1 << bits):
            continue
        freq = tile_eager.normalize_counts(counts, 1 << bits)
        assert freq.sum() == 1 << bits and np.all((freq > 0) == (counts > 0))
        cdfs, tables = tile_eager.tables_from_frequencies(freq[None], bits)
        symbols = tables[0] & 0xFF
        assert np.array_equal(np.bincount(symbols, minlength=256), freq.astype(np.int64))      # every slot maps into its symbol's range
        assert np.all((tables[0] >> 20) == cdfs[0][symbols])


def one_slot_at_a_time_in_numpy(counts: np.ndarray, table_size: int) -> np.ndarray:
    """The allocation written out with numpy, step for step as the reference's tile_ans/eager.py:17-60 computes it: what
    the C loop behind `tile_eager.normalize_counts` has to reproduce for every histogram, beyond the golden containers."""
    counts = np.asarray(counts, dtype=np.int64)
    present = np.flatnonzero(counts)
    share = counts.astype(np.float64) * (table_size / int(counts.sum()))
    freq = np.floor(share).astype(np.int64)
    freq[present] = np.maximum(freq[present], 1)
    gap = table_size - int(freq.sum())
    remainder = share - freq
    if gap > 0:
        key = np.full(counts.shape, np.inf)
        key[present] = -remainder[present]
        for _ in range(gap):
            symbol = int(np.argmin(key))
            freq[symbol] += 1
            key[symbol] += 1.0
    elif gap < 0:
        key = np.full(counts.shape, np.inf)
        pool = present[freq[present] > 1]
        if pool.size == 0:
            raise ValueError("unable to normalize rANS frequencies")
        key[pool] = remainder[pool]
        for _ in range(-gap):
            symbol = int(np.argmin(key))
            if not np.isfinite(key[symbol]):
                raise ValueError("unable to normalize rANS frequencies")
            freq[symbol] -= 1
            key[symbol] = key[symbol] + 1.0 if freq[symbol] > 1 else np.inf
    return freq.astype(np.uint16)


def test_normalised_frequencies_match_the_numpy_formulation():
    rng = np.random.default_rng(11)
    shortfalls = surpluses = 0
    for trial in range(1500):
        bits = int(rng.choice(tile_format.SUPPORTED_PROB_BITS))
        counts = np.zeros(256, dtype=np.int64)
        kind = trial % 4
        if kind == 0:
            present = rng.choice(256, size=rng.integers(1, 257), replace=False)
            counts[present] = rng.integers(1, 10 ** rng.integers(1, 8), size=present.size)
        elif kind == 1:                                  # a long tail of rare symbols under a few heavy ones: slots come back
            counts[:] = rng.integers(0, 3, size=256)
            counts[rng.integers(0, 256, size=4)] = rng.integers(10 ** 5, 10 ** 8, size=4)
        elif kind == 2:                                  # exact ties
            counts[rng.choice(256, size=rng.integers(2, 200), replace=False)] = int(rng.integers(1, 50))
        else:
            counts[:] = np.floor(rng.exponential(200.0, size=256)).astype(np.int64)
        if int(counts.sum()) == 0:
            counts[7] = 3
        try:
            want = one_slot_at_a_time_in_numpy(counts, 1 << bits)
        except ValueError:
            with pytest.raises(ValueError):
                tile_eager.normalize_counts(counts, 1 << bits)
            continue
        floors = int(np.maximum(np.floor(counts * ((1 << bits) / counts.sum())), counts > 0).sum())
        shortfalls += floors < (1 << bits)
        surpluses += floors > (1 << bits)
        assert np.array_equal(tile_eager.normalize_counts(counts, 1 << bits), want), (trial, bits, counts.tolist())
    assert shortfalls > 300 and surpluses > 100
    with pytest.raises(ValueError, match="empty"):
        tile_eager.normalize_counts(np.zeros(256, dtype=np.int64), 512)


def test_config_validation_and_defaults():
    from entropack_amd.schemes.config import validate_config
    validate_config(ep.TileANSConfig())
    for bad in (dict(probability_bits=8), dict(tile_elements=-1), dict(raw_lane_threshold=8.5), dict(threads_per_block=0)):
        with pytest.raises(ValueError):
            validate_config(ep.TileANSConfig(**bad))
    with pytest.raises(TypeError):
        validate_config(ep.TileANSConfig(tile_elements=1.5))
    from entropack_amd.registry import default_config
    config = default_config(torch.bfloat16)                    # the lossless scheme outranks the lossy one, as in the reference
    assert isinstance(config, ep.TileANSConfig) and (config.tile_elements, config.probability_bits) == (0, 11)
    assert default_config(torch.int32).tile_elements == 16384


def test_without_a_gpu_decoding_fails_loudly():
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    golden = TileGolden("bf16_300x200_auto")
    container = ep.CompressedTensor.unpack(torch.from_numpy(golden.quant_state.copy()))
    with pytest.raises((ep.DispatchError, RuntimeError)):
        ep.decompress(container, ep.TileANSConfig())
    with pytest.raises(ep.DispatchError):
        ep.decompress(container, ep.TileANSConfig(execution_backend="hip"))
