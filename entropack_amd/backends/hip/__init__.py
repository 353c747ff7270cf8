"""The `hip` backend: MI355X (gfx950) kernels in libentropack_hip.so, bound through its C ABI with ctypes.

This module plays the part the reference gives to its CuPy runtime glue (entropack/backends/cuda/__init__.py:4-16,
kernels.py:20-62, device.py:66-81): probing for a usable device, loading native code, and handing raw device
pointers and the current torch stream to it. Nothing here falls back to another implementation: when the library or
a gfx950 device is missing, `probe()` says why and every call raises.
"""
import ctypes
import os
import threading

import torch

_PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
LIBRARY_PATH = os.path.join(_PACKAGE_DIR, "libentropack_hip.so")
ABI_VERSION = 2

OK, EINVAL, EUNSUPPORTED, ERUNTIME, ENODEVICE, ETOOLARGE = range(6)
STATIC_ACCUMULATOR_FLOATS = 1 << 18          # EP_HIP_STATIC_ACCUMULATOR_FLOATS
TABLE_GLOBAL64, TABLE_LDS_BYTE, TABLE_LDS_WIDE, TABLE_LDS_RANK, TABLE_LDS_SYM = range(5)
TABLE_KIND_NAMES = {TABLE_GLOBAL64: "global64", TABLE_LDS_BYTE: "lds_byte", TABLE_LDS_WIDE: "lds_wide", TABLE_LDS_RANK: "lds_rank",
                    TABLE_LDS_SYM: "lds_sym"}
DECODE_ERRORS = {
    2: "a renormalisation read passed the start of a tile's payload (truncated or corrupt payload)",
    3: "a tile ended with unread payload words or a lane state other than 2**15 (corrupt payload, states or tables)",
    4: "offsets are not monotone or run past the payload",
}

#: torch dtype -> ep_hip_store_kind. The two fnuz float8 formats have no kernel; the lane decodes them via float32.
STORE_KINDS = {
    torch.float32: 0, torch.float16: 1, torch.float8_e4m3fn: 2, torch.float8_e5m2: 3, torch.int8: 4, torch.int16: 5,
    torch.int32: 6, torch.int64: 7, torch.uint8: 8, torch.uint16: 9, torch.uint32: 10, torch.uint64: 11, torch.bool: 12,
    torch.bfloat16: 13,
}


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("device", ctypes.c_int), ("compute_units", ctypes.c_int), ("lds_bytes_per_block", ctypes.c_int),
        ("wavefront_size", ctypes.c_int), ("is_gfx950", ctypes.c_int), ("arch", ctypes.c_char * 64),
    ]


class PlanDesc(ctypes.Structure):
    _fields_ = [
        ("table_kind", ctypes.c_int), ("prob_bits", ctypes.c_int), ("table_bytes", ctypes.c_size_t),
        ("lds_bytes", ctypes.c_int), ("max_alphabet", ctypes.c_int), ("alphabet_sum", ctypes.c_int),
        ("sym_offset", ctypes.c_int), ("present_offset", ctypes.c_int * 18), ("rank_values_half", ctypes.c_int),
    ]


class DecodeJob(ctypes.Structure):
    """ep_hip_decode_job: one container of a batched decode."""
    _fields_ = [
        ("payload_dev", ctypes.c_void_p), ("payload_words", ctypes.c_uint64), ("offsets_dev", ctypes.c_void_p),
        ("states_dev", ctypes.c_void_p), ("scales_dev", ctypes.c_void_p), ("tables_dev", ctypes.c_void_p),
        ("desc", ctypes.POINTER(PlanDesc)), ("out_offset", ctypes.c_uint64), ("store_kind", ctypes.c_int),
        ("tile_elements", ctypes.c_int), ("rows", ctypes.c_int64), ("cols_padded", ctypes.c_int64),
        ("error_dev", ctypes.c_void_p),
    ]


FUSED_SLOTS = 32                    # EP_HIP_FUSED_SLOTS


class FusedBatch(ctypes.Structure):
    """ep_hip_fused_batch: up to 32 tiles whose chains stay aligned in k (decode-to-GEMM through LDS)."""
    _fields_ = [("base", ctypes.c_int32), ("reserved", ctypes.c_int32 * 3), ("tile", ctypes.c_int32 * FUSED_SLOTS),
                ("delta", ctypes.c_int32 * FUSED_SLOTS)]


class HipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, call: str, status: int, detail: str):
        self.call, self.status = call, status
        super().__init__(f"{call} failed: {detail} (status {status})")


_SIGNATURES = {
    "ep_hip_abi_version": (ctypes.c_int, []),
    "ep_hip_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "ep_hip_last_runtime_error": (ctypes.c_int, []),
    "ep_hip_device_query": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(DeviceInfo)]),
    "ep_hip_plan_describe": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.POINTER(PlanDesc)]),
    "ep_hip_plan_build": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(PlanDesc), ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_decode_lattice": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.POINTER(PlanDesc), ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_decode_table_kind": (ctypes.c_int, [
        ctypes.POINTER(PlanDesc), ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int]),
    "ep_hip_decode_tile_ans": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
        ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_batch_plan": (ctypes.c_int, [
        ctypes.POINTER(DecodeJob), ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_size_t)]),
    "ep_hip_decode_lattice_batch": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_linear_fused_bf16": (ctypes.c_int, [
        ctypes.POINTER(DecodeJob), ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_linear_fused_bf16_static": (ctypes.c_int, [
        ctypes.POINTER(DecodeJob), ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "ep_hip_fused_plan": (ctypes.c_int, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int)]),
    "ep_hip_linear_fused_mfma_bf16": (ctypes.c_int, [
        ctypes.POINTER(DecodeJob), ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_linear_fused_mfma_i8": (ctypes.c_int, [
        ctypes.POINTER(DecodeJob), ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_linear_fused_mfma_workspace": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int64, ctypes.c_int]),
    "ep_hip_gemm_bf16": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
        ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "ep_hip_gemm_skinny_workspace": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]),
    "ep_hip_gemm_takes_small_blocks": (ctypes.c_int, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]),
    "ep_hip_gemm_i8_skinny": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
        ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
        ctypes.c_size_t, ctypes.c_void_p]),
    "ep_hip_gemm_bf16_skinny": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
        ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "ep_hip_gemm_i8": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
        ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "ep_hip_quantize_rows": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_void_p]),
    "ep_hip_rotate_quantize_rows": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_encode_quantize": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_encode_histogram": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_encode_row_scales": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_encode_rans": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_encode_offsets": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_encode_gather": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_tile_ans_histogram": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "ep_hip_tile_ans_encode": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)
FLOAT_KINDS = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

_library = None
_library_lock = threading.Lock()
_device_info: dict[int, DeviceInfo] = {}


def library() -> ctypes.CDLL:
    """The loaded C-ABI library. Raises (never substitutes anything) when it has not been built."""
    global _library
    if _library is None:
        with _library_lock:
            if _library is None:
                if not os.path.exists(LIBRARY_PATH):
                    raise ImportError(
                        f"{LIBRARY_PATH} is missing: build it with `python -m entropack_amd.build` (needs hipcc, gfx950)")
                lib = ctypes.CDLL(LIBRARY_PATH)
                for name, (restype, argtypes) in _SIGNATURES.items():
                    function = getattr(lib, name)
                    function.restype, function.argtypes = restype, argtypes
                if lib.ep_hip_abi_version() != ABI_VERSION:
                    raise ImportError(f"{LIBRARY_PATH} has ABI {lib.ep_hip_abi_version()}, this package needs {ABI_VERSION}")
                _library = lib
    return _library


def check(call: str, status: int) -> None:
    if status != OK:
        lib = library()
        detail = lib.ep_hip_error_string(status).decode()
        if status == ERUNTIME:
            detail += f", hipError_t {lib.ep_hip_last_runtime_error()}"
        raise HipError(call, status, detail)


def probe() -> str | None:
    """None when the backend can run here, otherwise the human-readable reason it cannot."""
    if not torch.cuda.is_available():
        return "torch.cuda.is_available() is False (no ROCm device / driver)"
    if getattr(torch.version, "hip", None) is None:
        return "this torch build is not a ROCm build"
    try:
        lib = library()
    except (ImportError, OSError) as error:
        return f"native library unavailable: {error}"
    info = DeviceInfo()
    status = lib.ep_hip_device_query(torch.cuda.current_device(), ctypes.byref(info))
    if status != OK:
        arch = info.arch.decode() or "unknown"
        return f"current device is {arch}, the kernels are built for gfx950 only"
    return None


def runs_on() -> torch.device:
    return torch.device("cuda", torch.cuda.current_device())


def device_info(index: int) -> DeviceInfo:
    info = _device_info.get(index)
    if info is None:
        info = DeviceInfo()
        check("ep_hip_device_query", library().ep_hip_device_query(index, ctypes.byref(info)))
        _device_info[index] = info
    return info


def pointer(tensor: torch.Tensor) -> int | None:
    """Raw device (or host) address; None for an empty tensor, whose data_ptr may be anything."""
    return tensor.data_ptr() if tensor.numel() else None


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
