"""`CompressedTensor`: a frozen tensor whose only real storage is one packed uint8 blob.

Blob layout (byte-identical to the reference's, entropack/compression/compressed_tensor.py:13-15,37-62, so that
checkpoints move freely between the two):

    bytes 0..7          little-endian u64: length L of the JSON header
    bytes 8..8+L        compact UTF-8 JSON with sorted keys: buffer_dtypes, buffer_names, buffer_shapes,
                        compress_method, dtype, header, shape
    zero padding        up to a multiple of 16
    buffer 0, padding   each buffer's raw bytes, each start aligned to 16, in `buffer_names` order
    ...                 the blob ends exactly at the aligned end of the last buffer

`buffers` are zero-copy typed views into the blob. The tensor reports the uncompressed shape and the dtype
`decompress` will return; `encoded_dtype` is the dtype the codec was given.
"""
import copy
import json
import math
from collections.abc import Mapping
from typing import Any

import torch
from torch.utils._python_dispatch import return_and_correct_aliasing

from ..registry import get_scheme
from ..schemes.base import HOST_MIRROR, HOST_MIRROR_LIMIT

ALIGNMENT = 16          # every component starts 16-byte aligned: the kernels read them with 16-byte loads
PREFIX_BYTES = 8
HEADER_KEYS = frozenset({"compress_method", "dtype", "shape", "buffer_names", "buffer_dtypes", "buffer_shapes", "header"})
DEFAULT_LEAF = "entropack_quant_state"


def _round_up(size: int) -> int:
    return (size + ALIGNMENT - 1) // ALIGNMENT * ALIGNMENT


def _dtype_to_name(dtype: torch.dtype) -> str:
    return str(dtype).split(".", 1)[1]


def _name_to_dtype(name) -> torch.dtype:
    if not isinstance(name, str) or not name:
        raise TypeError("CompressedTensor serialized dtype must be a non-empty string")
    found = getattr(torch, name, None)
    if not isinstance(found, torch.dtype):
        raise ValueError(f"Unsupported serialized torch dtype '{name}'")
    return found


def pack_quant_state(header: dict, buffers: Mapping[str, torch.Tensor], shape, encoded_dtype: torch.dtype) -> torch.Tensor:
    """Serialise header + buffers into one uint8 tensor on the buffers' device."""
    document = {
        "buffer_dtypes": [_dtype_to_name(t.dtype) for t in buffers.values()],
        "buffer_names": list(buffers),
        "buffer_shapes": [list(t.shape) for t in buffers.values()],
        "compress_method": header["compress_method"],
        "dtype": _dtype_to_name(encoded_dtype),
        "header": header,
        "shape": list(shape),
    }
    text = json.dumps(document, sort_keys=True, separators=(",", ":"), allow_nan=False).encode("utf-8")
    device = next(iter(buffers.values())).device
    cursor = _round_up(PREFIX_BYTES + len(text))
    placements = []
    for tensor in buffers.values():
        nbytes = tensor.numel() * tensor.element_size()
        placements.append((cursor, nbytes, tensor))
        cursor = _round_up(cursor + nbytes)
    blob = torch.zeros(cursor, dtype=torch.uint8, device=device)
    head = torch.frombuffer(bytearray(len(text).to_bytes(PREFIX_BYTES, "little") + text), dtype=torch.uint8)
    blob[: head.numel()].copy_(head)
    for start, nbytes, tensor in placements:
        if nbytes:
            blob[start:start + nbytes].copy_(tensor.detach().contiguous().reshape(-1).view(torch.uint8))
    return blob


def parse_quant_state(blob: torch.Tensor) -> tuple[dict, int]:
    """(JSON header, byte offset of the first buffer). Raises on anything that is not a well-formed blob."""
    if blob.dtype != torch.uint8 or blob.ndim != 1:
        raise TypeError(f"CompressedTensor quant_state must be a 1-D uint8 tensor; got {blob.dtype} with shape {tuple(blob.shape)}")
    total = blob.numel()
    if total < PREFIX_BYTES:
        raise ValueError(f"CompressedTensor quant_state is {total} bytes, too short to hold a header length")
    length = int.from_bytes(bytes(blob[:PREFIX_BYTES].detach().cpu().tolist()), "little")
    stop = PREFIX_BYTES + length
    if stop > total:
        raise ValueError(
            f"CompressedTensor header length {length} runs past the quant_state's end ({total} bytes); "
            "the checkpoint is likely truncated")
    try:
        document = json.loads(bytes(blob[PREFIX_BYTES:stop].detach().cpu().tolist()).decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as error:
        raise ValueError("CompressedTensor serialized header is invalid") from error
    if not isinstance(document, dict):
        raise TypeError("CompressedTensor serialized header is not a JSON object")
    absent = sorted(HEADER_KEYS - document.keys())
    if absent:
        raise ValueError(
            f"CompressedTensor serialized header is missing fields {absent}; "
            "it was likely written by a different entropack version")
    names = document["buffer_names"]
    repeated = sorted({name for name in names if names.count(name) > 1})
    if repeated:
        raise ValueError(f"CompressedTensor serialized header repeats buffers {repeated}")
    return document, _round_up(stop)


def buffer_views(blob: torch.Tensor, document: dict, start: int) -> dict[str, torch.Tensor]:
    views: dict[str, torch.Tensor] = {}
    cursor = start
    for name, dtype_name, shape in zip(document["buffer_names"], document["buffer_dtypes"], document["buffer_shapes"]):
        dtype = _name_to_dtype(dtype_name)
        nbytes = math.prod(shape) * dtype.itemsize
        if cursor + nbytes > blob.numel():
            raise ValueError(f"CompressedTensor quant_state is {blob.numel()} bytes, too short for buffer '{name}'")
        views[name] = blob[cursor:cursor + nbytes].view(dtype).view(shape)
        cursor = _round_up(cursor + nbytes)
    if cursor != blob.numel():
        raise ValueError(
            f"CompressedTensor quant_state is {blob.numel()} bytes, but its header and buffers account for "
            f"{cursor}; the entry is truncated or carries trailing bytes")
    return views


class CompressedTensor(torch.Tensor):
    """Compressed storage behind a (frozen) torch.Tensor face.

    Make one with :func:`compress` or :meth:`unpack`; get numbers back with :func:`decompress`. `to(dtype=...)`
    only changes what `decompress` returns and shares the blob; device moves move the blob. `state_dict()` /
    `from_state_dict()` and pickling all go through the blob, so `torch.save` keeps the compressed form and
    `torch.load(weights_only=True)` can read it back.
    """

    header: dict[str, Any]
    buffers: dict[str, torch.Tensor]
    entropack_quant_state: torch.Tensor

    @staticmethod
    def __new__(cls, header, buffers, shape, dtype, *, encoded_dtype=None):
        device = next(iter(buffers.values())).device
        return torch.Tensor._make_wrapper_subclass(cls, tuple(shape), dtype=dtype, device=device, requires_grad=False)

    def __init__(self, header, buffers, shape, dtype, *, encoded_dtype=None):
        self._bind(pack_quant_state(header, buffers, shape, dtype if encoded_dtype is None else encoded_dtype))

    @classmethod
    def _wrap(cls, blob: torch.Tensor, shape, dtype, parsed=None) -> "CompressedTensor":
        made = torch.Tensor._make_wrapper_subclass(cls, tuple(shape), dtype=dtype, device=blob.device, requires_grad=False)
        made._bind(blob, parsed)
        return made

    def _bind(self, blob: torch.Tensor, parsed=None) -> None:
        """`parsed` = (document, first buffer's offset) of a blob with the same bytes, already parsed and validated."""
        document, start = parse_quant_state(blob) if parsed is None else parsed
        self.entropack_quant_state = blob
        self._parsed = (document, start)
        self.header = document["header"]
        self.encoded_dtype = _name_to_dtype(document["dtype"])
        self.buffers = buffer_views(blob, document, start)
        if parsed is None:
            self.validate()

    def _rewrap(self, transform, dtype=None) -> "CompressedTensor":
        """The same bytes in another tensor (a copy, another device, an alias): nothing is parsed again, which for a
        device blob would mean reading it back. Small metadata buffers that leave the host take a host copy along
        (`host_copy`), so that planning a decode does not read them back either."""
        twin = type(self)._wrap(transform(self.entropack_quant_state), self.shape, self.dtype if dtype is None else dtype, self._parsed)
        for name, view in twin.buffers.items():
            source = self.buffers[name]
            mirror = getattr(source, HOST_MIRROR, None)
            if mirror is None and source.device.type == "cpu" and view.device.type != "cpu" \
                    and source.numel() * source.element_size() <= HOST_MIRROR_LIMIT:
                mirror = source.detach().clone()
            if mirror is not None and view.device.type != "cpu":
                setattr(view, HOST_MIRROR, mirror)
        return twin

    @classmethod
    def unpack(cls, quant_state: torch.Tensor) -> "CompressedTensor":
        """Rebuild a container around a packed blob, sharing its storage."""
        document, _ = parse_quant_state(quant_state)
        return cls._wrap(quant_state, document["shape"], _name_to_dtype(document["dtype"]))

    # -- tensor protocol ------------------------------------------------------------------------------------

    def __repr__(self) -> str:
        return (f"{type(self).__name__}(shape={tuple(self.shape)}, dtype={self.dtype}, device={self.device}, "
                f"scheme={self.compress_method!r})")

    def __tensor_flatten__(self):
        return ["entropack_quant_state"], ()

    @classmethod
    def __tensor_unflatten__(cls, inner_tensors, metadata, outer_size, outer_stride):
        return cls.unpack(inner_tensors["entropack_quant_state"])

    def __getstate__(self):
        return {"entropack_quant_state": self.entropack_quant_state}

    def __setstate__(self, state):
        self._bind(state["entropack_quant_state"])

    def __copy__(self):
        twin = self._rewrap(lambda blob: blob)
        if getattr(self, "_is_param", False):
            twin._is_param = True
        return twin

    def __deepcopy__(self, memo):
        if id(self) in memo:
            return memo[id(self)]
        twin = self._rewrap(lambda blob: copy.deepcopy(blob, memo))
        if getattr(self, "_is_param", False):
            twin._is_param = True
        memo[id(self)] = twin
        return twin

    def to(self, *args, copy: bool = False, **kwargs) -> "CompressedTensor":
        """Move the blob and/or change the dtype `decompress` returns. `copy` is keyword-only."""
        device, dtype, non_blocking, memory_format = torch._C._nn._parse_to(*args, **kwargs)
        moved = super().to(device=device, dtype=dtype, non_blocking=non_blocking, copy=copy, memory_format=memory_format)
        if copy and moved.device == self.device:
            return moved.clone()
        return moved

    def requires_grad_(self, requires_grad: bool = False):
        if requires_grad:
            raise RuntimeError("CompressedTensor cannot require gradients; decompress it to train dense values")
        return torch.Tensor.requires_grad_(self, False)

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        aten = torch.ops.aten
        subject = args[0] if args else None
        if func in (aten.detach.default, aten.alias.default):
            return return_and_correct_aliasing(func, args, kwargs, subject._rewrap(torch.detach))
        if func is aten.clone.default or func is aten._to_copy.default:
            if kwargs.get("memory_format") not in (None, torch.preserve_format, torch.contiguous_format):
                raise ValueError("CompressedTensor does not support that memory format")
            if func is aten.clone.default:
                return subject._rewrap(torch.clone)
            if kwargs.get("layout", torch.strided) not in (None, torch.strided):
                raise ValueError("CompressedTensor only supports strided storage")
            moves = {key: kwargs[key] for key in ("device", "non_blocking") if key in kwargs}
            return subject._rewrap(lambda blob: blob.to(**moves), dtype=kwargs.get("dtype"))
        lowered = func.decompose(*args, **kwargs)
        if lowered is not NotImplemented:
            return lowered
        raise NotImplementedError(f"CompressedTensor does not implement {func}; decompress it before numerical operations")

    # -- container facts ------------------------------------------------------------------------------------

    @property
    def compress_method(self) -> str:
        return self.header["compress_method"]

    @property
    def scheme(self):
        return get_scheme(self.compress_method)

    @property
    def lossless(self) -> bool:
        return self.scheme.lossless

    @property
    def actual_bpp(self) -> float:
        """Stored bits per element of `shape`, JSON header included."""
        return 8 * self.storage_nbytes() / math.prod(self.shape)

    def storage_nbytes(self, include_header: bool = True) -> int:
        total = self.entropack_quant_state.numel()
        return total if include_header else total - self._parsed[1]

    def validate(self) -> None:
        """Scheme known, dtype supported, buffer names as the scheme expects. Contents are not inspected."""
        if any(isinstance(value, CompressedTensor) for value in self.buffers.values()):
            raise TypeError("CompressedTensor buffers cannot contain another CompressedTensor")
        scheme = self.scheme
        if not scheme.supports(self.encoded_dtype):
            raise ValueError(f"'{scheme.name}' does not support format {self.encoded_dtype}")
        if set(self.buffers) != set(scheme.buffer_names):
            raise ValueError(
                f"CompressedTensor buffers for {self.compress_method} must be {list(scheme.buffer_names)}, got {sorted(self.buffers)}")

    def state_dict(self, leaf: str | None = None) -> dict[str, torch.Tensor]:
        self.validate()
        return {leaf or DEFAULT_LEAF: self.entropack_quant_state.detach()}

    @classmethod
    def from_state_dict(cls, state: Mapping[str, torch.Tensor], leaf: str | None = None) -> "CompressedTensor":
        leaf = leaf or DEFAULT_LEAF
        if leaf not in state:
            raise ValueError(f"CompressedTensor state is missing '{leaf}'")
        return cls.unpack(state[leaf])
