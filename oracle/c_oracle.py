"""ctypes binding of liblattice_oracle.so (the C twin of lattice_oracle.py) -- TEST INFRASTRUCTURE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblattice_oracle.so")
_lib = None

KINDS = {
    "float32": (0, np.float32), "float16": (1, np.uint16), "int8": (4, np.int8), "int16": (5, np.int16),
    "int32": (6, np.int32), "int64": (7, np.int64), "uint8": (8, np.uint8), "uint16": (9, np.uint16),
    "uint32": (10, np.uint32), "uint64": (11, np.uint64), "bool": (12, np.uint8), "bfloat16": (100, np.uint16),
}
ERRORS = {1: "bad argument", 2: "payload truncated", 3: "tile not fully consumed", 4: "bad frequency table"}


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, capture_output=True)
    return _LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        p = ctypes.c_void_p
        lib.orc_build_slot_table.argtypes = [p, ctypes.c_int, ctypes.c_int, p]
        lib.orc_decode_symbols.argtypes = [p, p, p, p, p, ctypes.c_int, ctypes.c_int, ctypes.c_int64, p, p, ctypes.c_int]
        lib.orc_reconstruct.argtypes = [p, p, p, p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, p, ctypes.c_int]
        lib.orc_decode.argtypes = [p, p, p, p, p, p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, p, ctypes.c_int]
        for fn in (lib.orc_build_slot_table, lib.orc_decode_symbols, lib.orc_reconstruct, lib.orc_decode):
            fn.restype = ctypes.c_int
        _lib = lib
    return _lib


def _ptr(array: np.ndarray):
    return array.ctypes.data_as(ctypes.c_void_p)


def _prep(buffers: dict):
    return {
        "payload": np.ascontiguousarray(buffers["payload"]).view(np.uint16) if np.asarray(buffers["payload"]).size else np.zeros(1, np.uint16),
        "offsets": np.ascontiguousarray(buffers["offsets"]).astype(np.uint32),
        "states": np.ascontiguousarray(buffers["states"]).astype(np.uint32),
        "stream_meta": np.ascontiguousarray(buffers["stream_meta"]).astype(np.int32),
        "freq_tables": np.ascontiguousarray(buffers["freq_tables"]).astype(np.uint16),
        "scales": np.ascontiguousarray(buffers["scales"]).astype(np.float32),
    }


def _check(rc: int) -> None:
    if rc:
        raise ValueError(f"lattice oracle: {ERRORS.get(rc, rc)}")


def build_slot_table(freq, prob_bits: int) -> np.ndarray:
    freq = np.ascontiguousarray(freq, dtype=np.uint16)
    lut = np.zeros(1 << prob_bits, dtype=np.uint64)
    _check(load().orc_build_slot_table(_ptr(freq), int(freq.size), int(prob_bits), _ptr(lut)))
    return lut


def decode_symbols(buffers: dict, prob_bits: int, tile_vectors: int, num_vectors: int, threads: int = 1):
    b = _prep(buffers)
    cosets = np.empty(num_vectors, dtype=np.int32)
    fields = np.empty((num_vectors, 8), dtype=np.int32)
    _check(load().orc_decode_symbols(
        _ptr(b["payload"]), _ptr(b["offsets"]), _ptr(b["states"]), _ptr(b["stream_meta"]), _ptr(b["freq_tables"]),
        int(prob_bits), int(tile_vectors), int(num_vectors), _ptr(cosets), _ptr(fields), int(threads)))
    return cosets, fields


def decode(buffers: dict, shape, dtype: str, threads: int = 1) -> np.ndarray:
    """Dense [rows, padded cols] in the container dtype (bf16/f16 as uint16 bit patterns, bool as uint8)."""
    b = _prep(buffers)
    cols, prob_bits, tile_elements = (int(v) for v in np.asarray(buffers["layout"]).reshape(-1))
    rows = int(shape[0])
    kind, np_dtype = KINDS[dtype]
    out = np.empty((rows, cols), dtype=np_dtype)
    _check(load().orc_decode(
        _ptr(b["payload"]), _ptr(b["offsets"]), _ptr(b["states"]), _ptr(b["stream_meta"]), _ptr(b["freq_tables"]),
        _ptr(b["scales"]), rows, cols, prob_bits, tile_elements, kind, _ptr(out), int(threads)))
    return out


# ---- tile_ans (lossless) ---------------------------------------------------------------------------------------------

_TILE_LIB_PATH = os.path.join(_HERE, "libtile_ans_oracle.so")
_tile_lib = None
TILE_ERRORS = {1: "bad argument", 2: "payload truncated", 3: "payload contains unread words", 4: "raw lane payload length is invalid"}


def load_tile_ans():
    global _tile_lib
    if _tile_lib is None:
        if not os.path.exists(_TILE_LIB_PATH):
            build()
        lib = ctypes.CDLL(_TILE_LIB_PATH)
        p = ctypes.c_void_p
        lib.tao_decode.argtypes = [p, p, p, p, p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int64, p, ctypes.c_int]
        lib.tao_decode.restype = ctypes.c_int
        _tile_lib = lib
    return _tile_lib


def tile_ans_decode(buffers: dict, element_bytes: int, threads: int = 1) -> np.ndarray:
    """Storage bytes (uint8[elements * element_bytes]) of a tile_ans container given as numpy buffers."""
    payload = np.ascontiguousarray(buffers["payload"]).view(np.uint16) if np.asarray(buffers["payload"]).size else np.zeros(1, np.uint16)
    offsets = np.ascontiguousarray(buffers["offsets"]).astype(np.uint32)
    states = np.ascontiguousarray(buffers["states"]).astype(np.uint32).reshape(-1) if np.asarray(buffers["states"]).size else np.zeros(32, np.uint32)
    tables = np.ascontiguousarray(buffers["decode_tables"]).astype(np.uint32)
    modes = np.ascontiguousarray(buffers["lane_modes"]).astype(np.uint8)
    tile_elements, prob_bits, lanes, elements = (int(v) for v in np.asarray(buffers["layout"]))
    if lanes != element_bytes:
        raise ValueError("layout does not match the element size")
    out = np.empty(elements * lanes, dtype=np.uint8)
    rc = load_tile_ans().tao_decode(_ptr(payload), _ptr(offsets), _ptr(states), _ptr(tables), _ptr(modes), tile_elements, prob_bits, lanes,
                                    elements, _ptr(out), int(threads))
    if rc:
        raise ValueError(f"tile_ans oracle: {TILE_ERRORS.get(rc, rc)}")
    return out
