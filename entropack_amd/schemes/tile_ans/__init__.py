"""The `tile_ans` scheme: lossless byte-lane coding, each lane raw or 32-way interleaved rANS over 256-symbol tables."""
import torch

from ..base import Scheme, packed_buffers, register_scheme
from .format import OPTIONS_BY_DTYPE, PACKED_KEYS, TileANSConfig, TileBuffers, validate_packed

__all__ = ["TileANSConfig", "TileANSScheme"]

LARGE_TENSOR_BYTES = 32 * 1024 * 1024


class TileANSScheme(Scheme):
    """Same public behaviour as the reference scheme (entropack/schemes/tile_ans/__init__.py:8-52), with a `hip` lane
    for decoding on MI355X and an `eager` lane that encodes on the CPU."""

    name = "tile_ans"
    buffer_names = PACKED_KEYS
    priority = 100
    dtypes = tuple(OPTIONS_BY_DTYPE)
    lanes = {"hip": "hip", "eager": "eager"}

    def options_for(self, dtype):
        tile_elements, probability_bits = OPTIONS_BY_DTYPE[dtype]
        return {"tile_elements": tile_elements, "probability_bits": probability_bits,
                "raw_lane_threshold": TileANSConfig().raw_lane_threshold}

    def encode(self, weight: torch.Tensor, config: TileANSConfig) -> dict:
        if weight.numel() == 0:
            raise ValueError(f"{self.name} does not support empty tensors")
        weight = weight.contiguous()
        tile_elements = config.tile_elements
        if tile_elements == 0:
            tile_elements = 4096 if weight.numel() * weight.element_size() <= LARGE_TENSOR_BYTES else 8192
        home = weight.device
        lane, lane_device = self.lane_for(weight, config.execution_backend)
        if lane_device is not None and home != lane_device:
            weight = weight.to(lane_device)
        buffers = lane.encode(weight=weight, tile_elements=tile_elements, probability_bits=config.probability_bits,
                              raw_lane_threshold=config.raw_lane_threshold, threads_per_block=config.threads_per_block)
        return {key: value.to(home) for key, value in buffers._asdict().items()}

    def validate_buffers(self, buffers, shape, dtype):
        validate_packed(buffers, shape, dtype)

    def decode(self, packed: dict, *, shape, dtype: torch.dtype, config: TileANSConfig) -> torch.Tensor:
        buffers = packed_buffers(packed, TileBuffers)
        home = buffers.layout.device
        lane, lane_device = self.lane_for(buffers.layout, config.execution_backend, gate_dtype=False)
        if lane_device is not None and home != lane_device:
            buffers = TileBuffers._make(value.to(lane_device) for value in buffers)
        out = lane.decode(buffers, dtype=dtype, threads_per_block=config.threads_per_block).reshape(shape)
        return out if out.device == home else out.to(home)


register_scheme(TileANSScheme())
