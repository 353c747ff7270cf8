"""CPU oracle for the lossless `tile_ans` decode -- TEST INFRASTRUCTURE, not product code.

A literal restatement (numpy arrays, per-symbol Python loops) of what the reference's CPU lane does, for small
inputs; `tile_ans_oracle.c` is its fast twin. Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
may import this module.

What each function follows in the reference (paths relative to the reference root):
  decode_group     entropack/schemes/tile_ans/eager.py:231-255  (table step, shared renormalisation)
  decode           entropack/schemes/tile_ans/eager.py:258-307  (stream order, raw lanes, tail group first)
  entry layout     entropack/schemes/tile_ans/eager.py:61-67    (cdf << 20 | freq << 8 | symbol, 4096 stored as 0)

Pinning: tests/test_tile_ans_golden.py checks `decode` against every fixture the reference wrote
(tests/golden/tile_ans/), including all-raw and all-coded lanes, tiles shorter than 32 elements, a single-symbol table
at prob_bits 12 (the frequency escape) and 1-, 2-, 4- and 8-byte elements; truncated and over-long payloads must
raise. Nothing here is "parity unpinned".
"""
import numpy as np

NUM_STATES = 32
STATE_MIN = 1 << 15
LANE_ANS, LANE_RAW = 0, 1


def decode_group(states, table, words, pointer, out, base, valid, prob_bits):
    """One symbol from each of the first `valid` states; the states that fell below 2**15 then read one word each,
    in ascending lane order, from the `count` words ending at `pointer`. Returns the new pointer."""
    size = 1 << prob_bits
    readers = []
    for lane in range(valid):
        x = int(states[lane])
        slot = x & (size - 1)
        entry = int(table[slot])
        freq = (entry >> 8) & 0xFFF
        if freq == 0:
            freq = size
        out[base + lane] = entry & 0xFF
        x = freq * (x >> prob_bits) + slot - (entry >> 20)
        states[lane] = x
        if x < STATE_MIN:
            readers.append(lane)
    first = pointer - len(readers)
    if first < 0:
        raise ValueError("tile_ans payload is truncated")
    for i, lane in enumerate(readers):
        states[lane] = (int(states[lane]) << 16) | int(words[first + i])
    return first


def decode(buffers: dict, element_bytes: int) -> np.ndarray:
    """The tensor's storage bytes, uint8[elements * element_bytes]."""
    payload = np.asarray(buffers["payload"]).view(np.uint16)
    offsets = np.asarray(buffers["offsets"]).astype(np.int64)
    states = np.asarray(buffers["states"]).astype(np.uint32)
    tables = np.asarray(buffers["decode_tables"]).astype(np.uint32)
    modes = np.asarray(buffers["lane_modes"]).astype(np.uint8)
    tile_elements, prob_bits, lanes, elements = (int(v) for v in np.asarray(buffers["layout"]))
    if lanes != element_bytes:
        raise ValueError("layout does not match the element size")
    tiles = -(-elements // tile_elements)
    out = np.empty(elements * lanes, dtype=np.uint8)
    stream = coded = 0
    for lane in range(lanes):
        for tile in range(tiles):
            first = tile * tile_elements
            count = min(tile_elements, elements - first)
            words = payload[offsets[stream]:offsets[stream + 1]]
            piece = np.empty(count, dtype=np.uint8)
            if modes[lane] == LANE_RAW:
                if words.size != (count + 1) // 2:
                    raise ValueError("tile_ans raw lane payload length is invalid")
                piece[0::2] = words & 0xFF
                piece[1::2] = words[:count // 2] >> 8
            else:
                x = states[coded].copy()
                coded += 1
                pointer = words.size
                rem = count % NUM_STATES
                at = count - rem
                if rem:
                    pointer = decode_group(x, tables[lane], words, pointer, piece, at, rem, prob_bits)
                while at > 0:
                    at -= NUM_STATES
                    pointer = decode_group(x, tables[lane], words, pointer, piece, at, NUM_STATES, prob_bits)
                if pointer != 0:
                    raise ValueError("tile_ans payload contains unread words")
            out[first * lanes + lane:(first + count) * lanes:lanes] = piece
            stream += 1
    return out
