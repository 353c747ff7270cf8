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
