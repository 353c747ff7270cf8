"""The `lattice_rans` scheme: E8-lattice vector quantisation entropy-coded with tiled, 32-way interleaved rANS.

Public behaviour of the reference scheme (entropack/schemes/lattice_rans/__init__.py:13-58): 2-D inputs of the
supported dtypes, columns padded to whole 8-vectors for the lane and cut back after decoding, buffers returned on the
device the input came from. Lanes here: `hip` decodes and encodes on an MI355X, `eager` encodes on the CPU.
"""
import torch

from ..base import Scheme, packed_buffers, register_scheme
from . import format as _format
from .format import EntroPackLossyConfig, LatticeBuffers, LatticeRANSConfig

__all__ = ["EntroPackLossyConfig", "LatticeRANSConfig", "LatticeRANSScheme"]

#: config fields handed to a lane's `encode` unchanged
_PASSED_ON = ("row_rdo_iterations", "row_rdo_candidates", "scale_search_iterations", "scale_search_max_vectors")


def _moved(buffers: LatticeBuffers, device) -> LatticeBuffers:
    if device is None or buffers.layout.device == device:
        return buffers
    return LatticeBuffers(*(tensor.to(device) for tensor in buffers))


class LatticeRANSScheme(Scheme):
    name = "lattice_rans"
    buffer_names = _format.PACKED_KEYS
    lossless = False
    dtypes = _format.SUPPORTED_DTYPES
    lanes = {"hip": "hip", "eager": "eager"}

    def _refuse(self, what: str):
        raise ValueError(f"{self.name} {what}")

    def _check_input(self, weight: torch.Tensor) -> None:
        if weight.dtype not in self.dtypes:
            self._refuse(f"does not support dtype {weight.dtype}")
        if weight.ndim != 2:
            self._refuse(f"encode requires exactly 2D input, got {weight.ndim}D")
        if weight.numel() == 0:
            self._refuse("does not support empty tensors")
        if weight.dtype.is_floating_point and not torch.isfinite(weight.float()).all().item():
            self._refuse("input must contain only finite values")

    def encode(self, weight: torch.Tensor, config: EntroPackLossyConfig) -> dict:
        self._check_input(weight)
        origin = weight.device
        bits_per_element = 1.0 if weight.dtype == torch.bool else 8.0 * weight.element_size()
        rate = min(float(config.target_bpp), bits_per_element)              # no point in asking for more than the input holds
        rows, cols = weight.shape
        loose = cols % _format.LATTICE_DIM
        matrix = weight.contiguous()
        if loose:
            matrix = torch.nn.functional.pad(matrix, (0, _format.LATTICE_DIM - loose))
        lane, device = self.lane_for(matrix, config.execution_backend)
        if device is not None:
            matrix = matrix.to(device)
        options = {name: getattr(config, name) for name in _PASSED_ON}
        options["prob_bits"] = int(config.prob_bits) if config.prob_bits else None
        options["tile_elements"] = _format.recommended_tile_elements(rate) if config.tile_elements is None else int(config.tile_elements)
        packed = lane.encode(weight=matrix, target_bpp=rate, **options)
        return {key: tensor.to(origin) for key, tensor in zip(LatticeBuffers._fields, packed)}

    def validate_buffers(self, buffers, shape, dtype):
        _format.validate_packed(buffers, tuple(shape), dtype)

    def decode(self, packed: dict, *, shape, dtype: torch.dtype, config: EntroPackLossyConfig) -> torch.Tensor:
        held = packed_buffers(packed, LatticeBuffers)
        origin = held.layout.device
        lane, device = self.lane_for(held.layout, config.execution_backend, gate_dtype=False)
        dense = lane.decode(_moved(held, device), shape=shape, dtype=dtype, threads_per_block=config.threads_per_block,
                            l2_prefetch=config.l2_prefetch)
        if shape and tuple(dense.shape) != tuple(shape):                     # the lane returns the padded columns
            dense = dense[:shape[0], :shape[1]]
        return dense.to(origin) if dense.device != origin else dense


register_scheme(LatticeRANSScheme())
