from .api import BatchDecompressor, CompressionFallbackWarning, compress, decompress, decompress_many
from .compressed_tensor import CompressedTensor

__all__ = ["BatchDecompressor", "CompressedTensor", "CompressionFallbackWarning", "compress", "decompress", "decompress_many"]
