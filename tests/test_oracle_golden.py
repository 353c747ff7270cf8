"""The CPU oracle (Python and C twins) against the fixtures the reference itself wrote, and against torch casts."""
import numpy as np
import pytest
import torch

from oracle import c_oracle, lattice_oracle as orc
from conftest import Golden, golden_names


def _restored_as(golden, array):
    """Compare in the fixture's raw-bit domain."""
    expect = golden.restored_bits
    rows, cols = golden.shape
    got = np.asarray(array)[:rows, :cols]
    if golden.dtype == "float32":
        got = got.view(np.int32)
    elif golden.dtype in ("bfloat16", "float16"):
        got = got.view(np.int16)
    elif golden.dtype == "int8":
        got = got.view(np.uint8)
    return got, expect


def test_python_oracle_matches_reference_symbols_and_output(golden):
    if golden.name.startswith(("c1_", "hi_")):
        pytest.skip("covered by the C twin; the per-symbol Python loop takes too long here")
    dense, cosets, fields = orc.decode(golden.buffers, golden.shape, golden.dtype)
    assert np.array_equal(cosets, golden.cosets)
    assert np.array_equal(fields, golden.fields)
    got, expect = _restored_as(golden, dense)
    assert np.array_equal(got, expect)


def test_c_oracle_matches_reference_symbols_and_output(golden):
    geo = orc.geometry(golden.buffers["layout"], golden.shape[0])
    cosets, fields = c_oracle.decode_symbols(golden.buffers, geo["prob_bits"], geo["tile_vectors"], geo["vectors"], threads=2)
    assert np.array_equal(cosets, golden.cosets)
    assert np.array_equal(fields, golden.fields)
    dense = c_oracle.decode(golden.buffers, golden.shape, golden.dtype, threads=2)
    got, expect = _restored_as(golden, dense)
    assert np.array_equal(got, expect)


def test_c1_python_oracle_first_tile_only():
    """Config 1 through the literal Python loop, cut to its last tile (912 vectors) to stay fast."""
    g = Golden("c1_256x256_bf16_3p5")
    geo = orc.geometry(g.buffers["layout"], g.shape[0])
    tv, tiles = geo["tile_vectors"], geo["tiles"]
    last = tiles - 1
    freqs = orc.stream_frequencies(g.buffers["freq_tables"], g.buffers["stream_meta"].astype(np.int64))
    off = g.buffers["offsets"].astype(np.int64)
    count = geo["vectors"] - last * tv
    cosets, fields = orc.decode_symbols(
        g.buffers["payload"][off[last]:off[last + 1]], np.array([0, off[last + 1] - off[last]]), g.buffers["states"][last:last + 1],
        freqs, geo["prob_bits"], tv, count)
    assert np.array_equal(cosets, g.cosets[last * tv:])
    assert np.array_equal(fields, g.fields[last * tv:])


def test_slot_table_partitions_the_slot_range():
    rng = np.random.default_rng(5)
    for pb in (9, 11, 13):
        size = 1 << pb
        cuts = np.sort(rng.choice(np.arange(1, size), size=40, replace=False))
        freq = np.diff(np.concatenate([[0], cuts, [size]]))
        freq = np.insert(freq, 7, 0)       # a zero-frequency symbol is skipped
        sym, frq, cdf = orc.build_slot_table(freq, pb)
        for slot in rng.integers(0, size, 300):
            s = int(np.searchsorted(np.cumsum(freq), slot, side="right"))   # brute force: the range holding slot
            assert sym[slot] == s and frq[slot] == freq[s] and cdf[slot] == freq[:s].sum()
        lut = c_oracle.build_slot_table(freq, pb)
        assert np.array_equal(lut & 0xFFFF, sym.astype(np.uint64))
        assert np.array_equal((lut >> np.uint64(16)) & np.uint64(0xFFFF), frq.astype(np.uint64))
        assert np.array_equal(lut >> np.uint64(32), cdf.astype(np.uint64))
    single = c_oracle.build_slot_table(np.array([1 << 10]), 10)            # f == table size packs as 0
    assert np.all(single == 0)
    with pytest.raises(ValueError):
        orc.build_slot_table(np.array([3, 4]), 9)
    with pytest.raises(ValueError):
        c_oracle.build_slot_table(np.array([3, 4]), 9)


def test_lattice_points_closed_form_and_negative_parity():
    # brute force over small z, including negative sums: z7 = 2m + (sum z0..z6 mod 2), mod taken non-negative
    rng = np.random.default_rng(0)
    values = rng.integers(-9, 10, size=(500, 8))
    cosets = rng.integers(0, 2, size=500)
    points = orc.lattice_points(cosets, values)
    for v, c, p in zip(values, cosets, points):
        parity = sum(int(t) for t in v[:7]) % 2
        expect = [float(t) + 0.5 * c for t in v[:7]] + [2.0 * v[7] + parity + 0.5 * c]
        assert p.tolist() == expect
        twice = np.rint(2 * p).astype(np.int64)               # membership in E8 = D8 u (D8 + 1/2)
        assert np.all(twice % 2 == c) and ((twice - c) // 2).sum() % 2 == 0


def test_float_tail_matches_torch_casts():
    torch.manual_seed(3)
    points = (torch.randint(-40, 40, (4096, 8)).float() + 0.5 * torch.randint(0, 2, (4096, 1)).float())
    scales = torch.rand(4096) * 0.05 + 1e-4
    dense = (points * scales.unsqueeze(1))
    mine = orc.rescale(points.numpy(), scales.numpy(), 4096, 8)
    assert np.array_equal(mine.view(np.int32), dense.numpy().view(np.int32))
    assert np.array_equal(orc.snap(mine, "bfloat16").view(np.int16), dense.to(torch.bfloat16).view(torch.int16).numpy())
    assert np.array_equal(orc.snap(mine, "float16").view(np.int16), dense.to(torch.float16).view(torch.int16).numpy())
    wide = dense * 3000.0
    for name, dt in (("int8", torch.int8), ("uint8", torch.uint8), ("int16", torch.int16), ("int32", torch.int32)):
        info = torch.iinfo(dt)
        expect = wide.round().clamp(float(info.min), float(np.nextafter(np.float32(info.max + 1.0), np.float32(0)))).to(dt)
        assert np.array_equal(orc.snap(wide.numpy(), name), expect.numpy())
    # ties round to even, saturation at both ends
    ties = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.5, 300.0, -128.5, -129.5, -1e9], dtype=np.float32)
    assert orc.snap(ties, "int8").tolist() == [0, 2, 2, 0, -2, 126, 127, 127, -128, -128, -128]
    huge = np.array([3.4e38, -3.4e38, 1e30], dtype=np.float32)
    assert np.array_equal(orc.snap(huge, "bfloat16").view(np.int16),
                          torch.from_numpy(huge).clamp(-3.3895313892515355e38, 3.3895313892515355e38).to(torch.bfloat16).view(torch.int16).numpy())
    assert np.array_equal(orc.snap(np.array([1e6, -1e6], np.float32), "float16").view(np.uint16), np.array([0x7BFF, 0xFBFF], np.uint16))


def test_c_oracle_reconstruct_kinds_match_python_snap():
    g = Golden("outlier_128x256_bf16_4p0")
    for kind in ("float32", "float16", "bfloat16", "int8", "uint8", "int16", "int32", "bool"):
        scaled = dict(g.buffers)
        if kind not in ("float32", "float16", "bfloat16"):
            scaled["scales"] = g.buffers["scales"] * np.float32(900.0)     # push values across the int8/uint8 limits
        c_out = c_oracle.decode(scaled, g.shape, kind, threads=1)
        values = orc.restore_minima(g.cosets, g.fields, scaled["stream_meta"])
        dense = orc.rescale(orc.lattice_points(g.cosets, values), scaled["scales"], g.shape[0], int(scaled["layout"][0]))
        py_out = orc.snap(dense, kind)
        if kind == "float16":
            py_out = py_out.view(np.uint16)
        if kind == "bool":
            py_out = py_out.astype(np.uint8)
        assert np.array_equal(c_out, py_out), kind


def test_truncated_and_unread_payloads_raise():
    g = Golden("ragged_66x200_bf16_4p0")
    geo = orc.geometry(g.buffers["layout"], g.shape[0])
    cut = dict(g.buffers)
    cut["payload"] = g.buffers["payload"][40:]
    cut["offsets"] = np.array([0, g.buffers["offsets"][1] - 40], dtype=np.uint32)
    with pytest.raises(ValueError):
        c_oracle.decode_symbols(cut, geo["prob_bits"], geo["tile_vectors"], geo["vectors"])
    padded = dict(g.buffers)
    padded["payload"] = np.concatenate([np.zeros(3, np.uint16), g.buffers["payload"]])
    padded["offsets"] = np.array([0, g.buffers["offsets"][1] + 3], dtype=np.uint32)
    with pytest.raises(ValueError):
        c_oracle.decode_symbols(padded, geo["prob_bits"], geo["tile_vectors"], geo["vectors"])
    with pytest.raises(ValueError):
        orc.decode(padded, g.shape, g.dtype)


def test_golden_set_is_complete():
    assert len(golden_names()) == 17
