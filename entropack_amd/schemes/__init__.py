from ..registry import all_schemes
from .base import Scheme
from .config import CompressionConfig, RawConfig
from .lattice_rans import EntroPackLossyConfig, LatticeRANSConfig

__all__ = ["CompressionConfig", "EntroPackLossyConfig", "LatticeRANSConfig", "RawConfig", "Scheme", "all_schemes"]
