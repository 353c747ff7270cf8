"""`compress` / `decompress`: the tensor-level API (same contract as entropack/compression/api.py:18-76)."""
import logging
import warnings

import torch

from ..registry import DispatchError, get_scheme, name_for_config
from ..schemes.config import CompressionConfig, RawConfig, validate_config
from .compressed_tensor import CompressedTensor

log = logging.getLogger("entropack")


class CompressionFallbackWarning(RuntimeWarning):
    """`compress` stored the tensor uncompressed because the requested scheme could not encode it."""


def compress(tensor: torch.Tensor, config: CompressionConfig) -> CompressedTensor:
    """Encode `tensor` with the scheme `config` belongs to.

    Bad configs and backend dispatch failures raise. Any other encode failure yields a `raw` container plus a
    `CompressionFallbackWarning`; its header names the scheme that was asked for and why it failed.
    """
    if isinstance(tensor, CompressedTensor):
        raise TypeError("compress expects an uncompressed tensor; decompress the container before recompressing")
    scheme = get_scheme(name_for_config(config))
    validate_config(config)
    try:
        packed = scheme.encode(tensor, config)
    except DispatchError:
        raise
    except Exception as error:
        log.warning("%s could not encode a %s %s tensor, storing it uncompressed: %s",
                    scheme.name, tuple(tensor.shape), tensor.dtype, error)
        why = f"{type(error).__name__}: {error}"
        warnings.warn(
            f"entropack stored a {tuple(tensor.shape)} {tensor.dtype} tensor uncompressed, at "
            f"{tensor.element_size() * 8} bits per parameter: compress_method={scheme.name!r} failed with {why}",
            CompressionFallbackWarning, stacklevel=2)
        return CompressedTensor(
            header={"compress_method": "raw", "requested": scheme.name, "reason": why},
            buffers=get_scheme("raw").encode(tensor, RawConfig()), shape=tuple(tensor.shape), dtype=tensor.dtype)
    return CompressedTensor(header={"compress_method": scheme.name}, buffers=packed, shape=tuple(tensor.shape), dtype=tensor.dtype)


def decompress(compressed: CompressedTensor, config: CompressionConfig) -> torch.Tensor:
    """Decode a container: a tensor of its shape and dtype on the device that holds its buffers."""
    validate_config(config)
    dense = compressed.scheme.decode(
        compressed.buffers, shape=tuple(compressed.shape), dtype=compressed.encoded_dtype, config=config)
    return dense.to(compressed.dtype)


class BatchDecompressor:
    """`decompress` for a whole list of `lattice_rans` containers (a model's layers) in one pass on the hip lane.

    Planning happens once here; every call decodes all containers with a handful of launches and returns tensors with
    the containers' shapes and dtypes, views into one output arena. The reference has no counterpart: its callers
    decode layer by layer (entropack/linear/linear.py:125-130).
    """

    def __init__(self, containers, config: CompressionConfig):
        from ..schemes.base import packed_buffers
        from ..schemes.lattice_rans import hip as hip_lane
        from ..schemes.lattice_rans.format import LatticeBuffers
        validate_config(config)
        if config.execution_backend not in (None, "auto", "hip"):
            raise DispatchError(f"batched decode runs on the hip backend only, not {config.execution_backend!r}")
        self._containers = list(containers)
        items = []
        for compressed in self._containers:
            if compressed.compress_method != "lattice_rans":
                raise ValueError(f"batched decode handles lattice_rans containers, got {compressed.compress_method!r}")
            buffers = packed_buffers(compressed.buffers, LatticeBuffers)
            items.append((buffers, tuple(compressed.shape), compressed.encoded_dtype))
        self._decoder = hip_lane.BatchDecoder(items)
        self.arena_bytes = self._decoder.arena_bytes

    def __call__(self, arena: torch.Tensor | None = None) -> list[torch.Tensor]:
        outputs = []
        for compressed, dense in zip(self._containers, self._decoder.decode(arena)):
            rows, cols = compressed.shape
            if tuple(dense.shape) != (rows, cols):
                dense = dense[:rows, :cols]
            outputs.append(dense.to(compressed.dtype))
        return outputs

    def check_errors(self) -> None:
        self._decoder.check_errors()


def decompress_many(containers, config: CompressionConfig) -> list[torch.Tensor]:
    """Decode every container of a list in one device pass; see `BatchDecompressor` to reuse the plan."""
    return BatchDecompressor(containers, config)()
