"""The `tile_ans` scheme: lossless byte-lane coding, each lane raw or 32-way interleaved rANS over 256-symbol tables.

Public behaviour of the reference scheme (entropack/schemes/tile_ans/__init__.py:8-52): any tensor of a supported
dtype, flattened; `tile_elements = 0` means 4096, or 8192 above 32 MiB of storage; buffers come back on the device the
input was on. Lanes here: `hip` decodes and encodes on an MI355X, `eager` encodes on the CPU.
"""
import torch

from ..base import Scheme, packed_buffers, register_scheme
from . import format as _format
from .format import TileANSConfig, TileBuffers

__all__ = ["TileANSConfig", "TileANSScheme"]

#: storage size above which automatic tile selection doubles the tile
LARGE_TENSOR_BYTES = 32 << 20


def _automatic_tile(weight: torch.Tensor) -> int:
    return 8192 if weight.numel() * weight.element_size() > LARGE_TENSOR_BYTES else 4096


class TileANSScheme(Scheme):
    name = "tile_ans"
    buffer_names = _format.PACKED_KEYS
    priority = 100                                      # the default scheme for every dtype it stores
    dtypes = tuple(_format.OPTIONS_BY_DTYPE)
    lanes = {"hip": "hip", "eager": "eager"}

    def options_for(self, dtype):
        tile_elements, probability_bits = _format.OPTIONS_BY_DTYPE[dtype]
        defaults = TileANSConfig()
        return dict(tile_elements=tile_elements, probability_bits=probability_bits, raw_lane_threshold=defaults.raw_lane_threshold)

    def encode(self, weight: torch.Tensor, config: TileANSConfig) -> dict:
        if not weight.numel():
            raise ValueError(f"{self.name} does not support empty tensors")
        origin = weight.device
        lane, device = self.lane_for(weight, config.execution_backend)
        source = weight.contiguous() if device is None else weight.contiguous().to(device)
        packed = lane.encode(weight=source, tile_elements=config.tile_elements or _automatic_tile(weight),
                             probability_bits=config.probability_bits, raw_lane_threshold=config.raw_lane_threshold,
                             threads_per_block=config.threads_per_block)
        return {key: tensor.to(origin) for key, tensor in zip(TileBuffers._fields, packed)}

    def validate_buffers(self, buffers, shape, dtype):
        _format.validate_packed(buffers, shape, dtype)

    def decode(self, packed: dict, *, shape, dtype: torch.dtype, config: TileANSConfig) -> torch.Tensor:
        held = packed_buffers(packed, TileBuffers)
        origin = held.layout.device
        lane, device = self.lane_for(held.layout, config.execution_backend, gate_dtype=False)
        if device is not None and device != origin:
            held = TileBuffers(*(tensor.to(device) for tensor in held))
        restored = lane.decode(held, dtype=dtype, threads_per_block=config.threads_per_block).reshape(shape)
        return restored.to(origin) if restored.device != origin else restored


register_scheme(TileANSScheme())
