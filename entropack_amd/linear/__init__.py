from .ahead import DecodeAhead
from .linear import CompressedINT8Linear, CompressedLinear, QuantizedLinear

__all__ = ["CompressedINT8Linear", "CompressedLinear", "DecodeAhead", "QuantizedLinear"]
