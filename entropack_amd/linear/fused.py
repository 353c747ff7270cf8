"""Forward paths of the compressed linear layers that never call a library GEMM."""
import torch

from . import kernels


def linear_forward(layer, x: torch.Tensor) -> torch.Tensor:
    """Decode the weight with the HIP decode kernel and multiply on the matrix cores with this package's GEMM."""
    weight = layer.dequantize(x.device)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("the fused forward runs in bfloat16; use forward_mode='decode_then_gemm' for other dtypes")
    return kernels.gemm_bf16(x, weight, layer._bias_on(x.device), out_dtype=x.dtype)


def int8_linear_forward(layer, activation: torch.Tensor, activation_scale: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    codes = layer.codes(activation.device)
    return kernels.int8_gemm(activation, codes, activation_scale, layer._scale(codes.device), layer._bias_on(activation.device), out_dtype)
