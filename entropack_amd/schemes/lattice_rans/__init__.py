"""The `lattice_rans` scheme: E8-lattice vector quantisation entropy-coded with tiled, 32-way interleaved rANS."""
import torch

from ..base import Scheme, packed_buffers, register_scheme
from .format import (
    LATTICE_DIM, PACKED_KEYS, SUPPORTED_DTYPES, EntroPackLossyConfig, LatticeBuffers, LatticeRANSConfig,
    recommended_tile_elements, validate_packed,
)

__all__ = ["EntroPackLossyConfig", "LatticeRANSConfig", "LatticeRANSScheme"]


class LatticeRANSScheme(Scheme):
    """Same public behaviour as the reference scheme (entropack/schemes/lattice_rans/__init__.py:13-58), with a
    `hip` lane for decoding on MI355X and an `eager` lane that encodes on the CPU."""

    name = "lattice_rans"
    buffer_names = PACKED_KEYS
    lossless = False
    priority = 0
    dtypes = SUPPORTED_DTYPES
    lanes = {"hip": "hip", "eager": "eager"}

    def encode(self, weight: torch.Tensor, config: EntroPackLossyConfig) -> dict:
        if weight.dtype not in SUPPORTED_DTYPES:
            raise ValueError(f"{self.name} does not support dtype {weight.dtype}")
        if weight.ndim != 2:
            raise ValueError(f"{self.name} encode requires exactly 2D input, got {weight.ndim}D")
        if weight.numel() == 0:
            raise ValueError(f"{self.name} does not support empty tensors")
        if weight.dtype.is_floating_point and not bool(torch.isfinite(weight.float()).all()):
            raise ValueError(f"{self.name} input must contain only finite values")
        weight = weight.contiguous()
        width = 1.0 if weight.dtype == torch.bool else weight.element_size() * 8.0
        target_bpp = min(float(config.target_bpp), width)
        home = weight.device
        rows, cols = weight.shape
        pad = -cols % LATTICE_DIM
        if pad:
            weight = torch.cat([weight, weight.new_zeros(rows, pad)], dim=1)
        lane, lane_device = self.lane_for(weight, config.execution_backend)
        if lane_device is not None and weight.device != lane_device:
            weight = weight.to(lane_device)
        tile_elements = recommended_tile_elements(target_bpp) if config.tile_elements is None else int(config.tile_elements)
        packed = lane.encode(
            weight=weight, target_bpp=target_bpp, prob_bits=None if config.prob_bits in (None, 0) else int(config.prob_bits),
            tile_elements=tile_elements, row_rdo_iterations=config.row_rdo_iterations,
            row_rdo_candidates=config.row_rdo_candidates, scale_search_iterations=config.scale_search_iterations,
            scale_search_max_vectors=config.scale_search_max_vectors,
        )
        return {key: value.to(home) for key, value in packed._asdict().items()}

    def validate_buffers(self, buffers, shape, dtype):
        validate_packed(buffers, tuple(shape), dtype)

    def decode(self, packed: dict, *, shape, dtype: torch.dtype, config: EntroPackLossyConfig) -> torch.Tensor:
        buffers = packed_buffers(packed, LatticeBuffers)
        home = buffers.layout.device
        lane, lane_device = self.lane_for(buffers.layout, config.execution_backend, gate_dtype=False)
        if lane_device is not None and home != lane_device:
            buffers = LatticeBuffers._make(value.to(lane_device) for value in buffers)
        out = lane.decode(buffers, shape=shape, dtype=dtype, threads_per_block=config.threads_per_block,
                          l2_prefetch=config.l2_prefetch)
        if shape and tuple(out.shape) != tuple(shape):
            out = out[: shape[0], : shape[1]]
        return out if out.device == home else out.to(home)


register_scheme(LatticeRANSScheme())
