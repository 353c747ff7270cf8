"""entropack_amd: the lossy decode-and-matmul path of EntroPack, built for AMD Instinct MI355X (gfx950).

Drop-in names: `compress`, `decompress`, `CompressedTensor`, `EntroPackLossyConfig`, `TileANSConfig`, `CompressedLinear`,
`CompressedINT8Linear`; `BatchDecompressor` / `DecodeAhead` decode many layers per pass. Decoding runs on the `hip` backend only.
"""
from .compression import BatchDecompressor, CompressedTensor, CompressionFallbackWarning, compress, decompress, decompress_many
from .linear import CompressedINT8Linear, CompressedLinear, DecodeAhead
from .registry import DispatchError
from .schemes import CompressionConfig, EntroPackLossyConfig, LatticeRANSConfig, RawConfig, TileANSConfig

__version__ = "0.1.0"

__all__ = [
    "BatchDecompressor", "CompressedINT8Linear", "CompressedLinear", "CompressedTensor", "CompressionConfig", "CompressionFallbackWarning", "DecodeAhead", "DispatchError", "EntroPackLossyConfig",
    "LatticeRANSConfig", "RawConfig", "TileANSConfig", "__version__", "compress", "decompress", "decompress_many",
]
