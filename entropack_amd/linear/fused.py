"""Forward paths of the compressed linear layers that never call a library GEMM.

One to four activation rows (the memory-bound regime): the decode kernel multiplies every decoded vector with the
activations in registers, so the dense weight is neither written nor re-read. More rows: the weight is decoded once
and multiplied on the matrix cores with this package's GEMM; at that size the serial rANS chain of a tile, not memory
traffic, bounds the decode, and a multiply inside the decode kernel would only slow the GEMM down.
"""
import torch

from ..schemes.base import packed_buffers
from ..schemes.lattice_rans import hip as hip_lane
from ..schemes.lattice_rans.format import LatticeBuffers
from . import kernels


def linear_forward(layer, x: torch.Tensor) -> torch.Tensor:
    container = layer._container()
    if container.compress_method == "lattice_rans" and container.encoded_dtype == torch.bfloat16:
        on_device = container.to(device=x.device)
        buffers = packed_buffers(on_device.buffers, LatticeBuffers)
        if hip_lane.fused_linear_pays(buffers, tuple(container.shape), x):
            return hip_lane.linear_rows(buffers, shape=tuple(container.shape), x=x, bias=layer._bias_on(x.device))
    weight = layer._decoded_for(x)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("the fused forward runs in bfloat16; use forward_mode='decode_then_gemm' for other dtypes")
    return kernels.gemm_bf16(x, weight, layer._bias_on(x.device), out_dtype=x.dtype)


def int8_linear_forward(layer, activation: torch.Tensor, activation_scale: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    codes = layer._decoded_for(activation)
    return kernels.int8_gemm(activation, codes, activation_scale, layer._scale(codes.device), layer._bias_on(activation.device), out_dtype)
