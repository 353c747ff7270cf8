"""Compression schemes of this package: `lattice_rans` (lossy, the decode hot path), `tile_ans` (lossless) and `raw`.
Importing a scheme's package registers it."""
from . import base as _base
from . import config as _config
from . import lattice_rans as _lattice_rans
from . import tile_ans as _tile_ans
from ..registry import all_schemes

Scheme = _base.Scheme
CompressionConfig = _config.CompressionConfig
RawConfig = _config.RawConfig
LatticeRANSConfig = _lattice_rans.LatticeRANSConfig
EntroPackLossyConfig = _lattice_rans.EntroPackLossyConfig
TileANSConfig = _tile_ans.TileANSConfig

__all__ = ["CompressionConfig", "EntroPackLossyConfig", "LatticeRANSConfig", "RawConfig", "Scheme", "TileANSConfig", "all_schemes"]
