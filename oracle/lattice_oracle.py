"""CPU oracle for the lattice_rans decode path -- TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the shipped
package never does. It restates, in plain numpy and Python loops, what the reference's CPU lane computes when
it decodes one ``lattice_rans`` container:

    entropy decode   entropack/schemes/lattice_rans/rans.py:74-130,189-221
    field minima     entropack/schemes/lattice_rans/eager.py:355-367
    E8 point         entropack/schemes/lattice_rans/eager.py:54-58
    row rescale      entropack/schemes/lattice_rans/eager.py:370-376
    container snap   entropack/schemes/lattice_rans/format.py:153-168
    geometry         entropack/schemes/lattice_rans/format.py:171-189,283-291

The loop structure (one Python iteration per lane per symbol) deliberately mirrors the reference's eager lane,
so timing this module is the stand-in for "the reference's CPU path" on a machine the reference cannot reach.
A fast C twin of the same functions lives in lattice_oracle.c.

Pinning (see tests/test_oracle_golden.py): every function below is checked against fixtures written by the
reference itself (tests/golden/*.npz: symbol planes and dense output for 13 containers, bf16/f16/f32/int8,
prob_bits 9..13, ragged/padded/empty-payload/tiny-tile/wide-alphabet cases), and the float tail is checked
against torch's own casts. No function here is "parity unpinned".
"""
import numpy as np

NUM_STATES = 32          # entropack/schemes/tile_ans/format.py:19
STATE_MIN = 1 << 15      # entropack/schemes/tile_ans/format.py:20
LATTICE_DIM = 8          # entropack/schemes/lattice_rans/format.py:57
NUM_FIELDS = 8           # format.py:58
NUM_STREAMS = 17         # format.py:60  (1 coset stream + 8 fields x 2 cosets)
META_N, META_MIN, META_OFF, META_ALPHA = 0, 1, 2, 3   # format.py:75-79


def tile_vectors_of(tile_elements: int) -> int:
    """format.py:171-172 -- a tile of `tile_elements` symbols holds tile_elements // 9 vectors, at least 32."""
    return max(32, int(tile_elements) // 9)


def geometry(layout, rows: int) -> dict:
    """format.py:179-189,283-291 -- layout = (padded cols, prob_bits, tile_elements)."""
    cols, prob_bits, tile_elements = (int(v) for v in layout)
    if cols <= 0 or cols % LATTICE_DIM:
        raise ValueError("cols must be a positive multiple of 8")
    if prob_bits not in (9, 10, 11, 12, 13, 14, 15):
        raise ValueError(f"prob_bits {prob_bits} unsupported")
    if tile_elements <= 0:
        raise ValueError("tile_elements must be positive")
    tv = tile_vectors_of(tile_elements)
    vectors = int(rows) * (cols // LATTICE_DIM)
    return {"rows": int(rows), "cols": cols, "prob_bits": prob_bits, "tile_elements": tile_elements,
            "tile_vectors": tv, "vectors": vectors, "tiles": (vectors + tv - 1) // tv}


def stream_frequencies(freq_tables, meta):
    """eager.py:355-358 -- slice the concatenated frequency table by (freq_offset, alphabet)."""
    return [np.asarray(freq_tables[int(r[META_OFF]): int(r[META_OFF]) + int(r[META_ALPHA])], dtype=np.int64) for r in meta]


def build_slot_table(freq, prob_bits: int):
    """rans.py:74-95 -- slot -> (symbol, frequency, cdf) for one stream.

    Returns three int64 arrays of length 2**prob_bits. (The reference packs them into one u64 with a frequency
    of 2**prob_bits stored as 0; the unpacked triple is the same map.)
    """
    freq = np.asarray(freq, dtype=np.int64)
    size = 1 << prob_bits
    if freq.size > size:
        raise ValueError("alphabet exceeds table size")
    if int(freq.sum()) != size:
        raise ValueError("normalized frequencies must sum to table_size")
    sym = np.zeros(size, dtype=np.int64)
    frq = np.zeros(size, dtype=np.int64)
    cdf = np.zeros(size, dtype=np.int64)
    running = 0
    for symbol in range(freq.size):
        f = int(freq[symbol])
        if f == 0:
            continue
        sym[running:running + f] = symbol
        frq[running:running + f] = f
        cdf[running:running + f] = running
        running += f
    assert running == size
    return sym, frq, cdf


def _decode_step(states, tables, table_ids, words, pointer, out, valid_lanes, prob_bits):
    """rans.py:98-120 -- one symbol for each of the first `valid_lanes` lanes, then the shared renormalisation.

    Lanes whose state fell below 2**15 each take one 16-bit word; the i-th such lane in ascending lane order gets
    words[pointer - n + i], and the pointer drops by n.
    """
    mask = (1 << prob_bits) - 1
    readers = []
    for lane in range(valid_lanes):
        x = int(states[lane])
        slot = x & mask
        sym, frq, cdf = tables[0 if table_ids is None else int(table_ids[lane])]
        out[lane] = int(sym[slot])
        x = int(frq[slot]) * (x >> prob_bits) + slot - int(cdf[slot])
        states[lane] = x
        if x < STATE_MIN:
            readers.append(lane)
    first = pointer - len(readers)
    if first < 0:
        raise ValueError("rANS payload is truncated")
    for i, lane in enumerate(readers):
        states[lane] = (int(states[lane]) << 16) | int(words[first + i])
    return first


def _decode_group(tables, states, words, pointer, coset_out, field_out, valid_lanes, prob_bits):
    """rans.py:123-130 -- coset from stream 0, then field f from stream 1 + 2f + coset, f = 0..7."""
    pointer = _decode_step(states, [tables[0]], None, words, pointer, coset_out, valid_lanes, prob_bits)
    for f in range(NUM_FIELDS):
        pointer = _decode_step(states, [tables[1 + 2 * f], tables[2 + 2 * f]], coset_out, words, pointer,
                               field_out[:, f], valid_lanes, prob_bits)
    return pointer


def decode_symbols(payload, offsets, states, frequencies, prob_bits, tile_vectors, num_vectors, check_final_states=True):
    """rans.py:189-221 -- all tiles; per tile the partial tail group first, then full groups downwards.

    Returns (cosets int64[V], shifted fields int64[V, 8]). Raises when a tile leaves payload words unread
    (rans.py:219-220); with `check_final_states` also when a lane does not end at 2**15, which the device
    decoders of the reference treat as the same error (lattice_rans.cu:799,933,1090).
    """
    tables = [None if np.asarray(f).size == 0 else build_slot_table(f, prob_bits) for f in frequencies]
    cosets = np.empty(num_vectors, dtype=np.int64)
    fields = np.empty((num_vectors, NUM_FIELDS), dtype=np.int64)
    tiles = max(1, (num_vectors + tile_vectors - 1) // tile_vectors)
    for tile in range(tiles):
        begin = tile * tile_vectors
        count = min(tile_vectors, num_vectors - begin)
        words = np.asarray(payload[int(offsets[tile]):int(offsets[tile + 1])], dtype=np.uint16)
        x = [int(v) for v in np.asarray(states[tile], dtype=np.uint32)]
        pointer = int(words.size)
        rem = count % NUM_STATES
        off = count - rem
        if rem:
            pointer = _decode_group(tables, x, words, pointer, cosets[begin + off:begin + count],
                                    fields[begin + off:begin + count], rem, prob_bits)
        while off > 0:
            off -= NUM_STATES
            pointer = _decode_group(tables, x, words, pointer, cosets[begin + off:begin + off + NUM_STATES],
                                    fields[begin + off:begin + off + NUM_STATES], NUM_STATES, prob_bits)
        if pointer != 0:
            raise ValueError("tile leaves unread payload words")
        if check_final_states and any(v != STATE_MIN for v in x):
            raise ValueError("tile does not end in the initial encoder state")
    return cosets, fields


def restore_minima(cosets, shifted_fields, meta):
    """eager.py:361-367 -- field f of a coset-c vector was stored minus stream_meta[1 + 2f + c].sym_min."""
    meta = np.asarray(meta, dtype=np.int64)
    values = np.array(shifted_fields, dtype=np.int64, copy=True)
    for f in range(NUM_FIELDS):
        values[:, f] += np.where(cosets == 0, meta[1 + 2 * f, META_MIN], meta[2 + 2 * f, META_MIN])
    return values


def lattice_points(cosets, values):
    """eager.py:54-58 -- z0..z6 as stored; z7 = 2 m + parity(z0 + .. + z6); point = z + c / 2, in float32."""
    z = np.array(values, dtype=np.int64, copy=True)
    parity = np.remainder(z[:, :7].sum(axis=1), 2)     # non-negative, like torch.remainder
    z[:, 7] = 2 * z[:, 7] + parity
    return z.astype(np.float32) + np.float32(0.5) * cosets.astype(np.float32)[:, None]


def rescale(points, scales, rows, cols):
    """eager.py:370-376 -- one float32 multiply (round to nearest) by the row's scale."""
    per_vector = np.repeat(np.asarray(scales, dtype=np.float32), cols // LATTICE_DIM)
    return (points * per_vector[:, None]).astype(np.float32).reshape(rows, cols)


def f32_to_bf16_bits(values):
    """Round-to-nearest-even float32 -> bfloat16, as the bit pattern (uint16). NaN keeps a quiet payload."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, ((bits >> 16) | 0x40).astype(np.uint16), rounded)


_INT_RANGES = {
    "int8": (np.int8, -128.0, 128.0), "int16": (np.int16, -32768.0, 32768.0),
    "int32": (np.int32, -2147483648.0, 2147483648.0), "int64": (np.int64, -9223372036854775808.0, 9223372036854775808.0),
    "uint8": (np.uint8, 0.0, 256.0), "uint16": (np.uint16, 0.0, 65536.0),
    "uint32": (np.uint32, 0.0, 4294967296.0), "uint64": (np.uint64, 0.0, 18446744073709551616.0),
}


def snap(values, dtype: str):
    """format.py:153-168 -- cast the float32 reconstruction into the container dtype, saturating.

    float32: identity. bfloat16/float16: clamp to +-largest finite, round to nearest even (bfloat16 is returned as
    its uint16 bit pattern; numpy has no such type). Integers: round half to even, clamp to
    [min, nextafter(max + 1, 0)], truncate. bool: rint != 0.
    """
    values = np.asarray(values, dtype=np.float32)
    if dtype == "float32":
        return values
    if dtype == "bfloat16":
        limit = np.float32(3.3895313892515355e38)
        return f32_to_bf16_bits(np.clip(values, -limit, limit))
    if dtype == "float16":
        return np.clip(values, np.float32(-65504.0), np.float32(65504.0)).astype(np.float16)
    if dtype == "bool":
        return np.rint(values) != 0
    if dtype in _INT_RANGES:
        kind, low, high_exclusive = _INT_RANGES[dtype]
        high = np.nextafter(np.float32(high_exclusive), np.float32(0.0))
        clamped = np.clip(np.rint(values), np.float32(low), high)
        if kind in (np.int64, np.uint64):
            return np.array([int(v) for v in clamped.reshape(-1)], dtype=kind).reshape(clamped.shape)
        return clamped.astype(kind)
    raise ValueError(f"no snap rule for {dtype}")


def decode(buffers: dict, shape, dtype: str):
    """eager.py:379-396 -- the whole CPU decode of one container.

    `buffers` maps the seven names (payload, offsets, states, stream_meta, freq_tables, scales, layout) to numpy
    arrays. Returns (dense [rows, padded cols] in the container dtype -- bf16 as uint16 bits --, cosets, fields).
    """
    geo = geometry(buffers["layout"], shape[0])
    meta = np.asarray(buffers["stream_meta"], dtype=np.int64).reshape(NUM_STREAMS, 4)
    freqs = stream_frequencies(np.asarray(buffers["freq_tables"]), meta)
    cosets, shifted = decode_symbols(
        np.asarray(buffers["payload"]), np.asarray(buffers["offsets"], dtype=np.int64),
        np.asarray(buffers["states"]).reshape(-1, NUM_STATES), freqs, geo["prob_bits"], geo["tile_vectors"], geo["vectors"],
    )
    values = restore_minima(cosets, shifted, meta)
    dense = rescale(lattice_points(cosets, values), buffers["scales"], geo["rows"], geo["cols"])
    return snap(dense, dtype), cosets, shifted
