"""`forward_mode="fused"` and `"fused_through_lds"` of the compressed linear layers: what runs for how many activation rows.

"fused":

  rows M            weight written to memory?   kernels
  1 (and 2..4 on    no                          the decode kernel multiplies every decoded vector with the activations in
  weights large                                 registers (`ep_hip_linear_fused_bf16`, two bf16 products per instruction):
  enough that their                             the memory-bound regime, where the dense weight would be 16 / bpp times the
  decode is bound by                            bytes of the container
  throughput)
  up to 128         yes, once                   decode, then this package's split-K skinny product (`ep_hip_gemm_bf16_skinny`),
                                                which streams the weight at 75 % of the memory bandwidth
  more              yes, once                   decode, then a tiled product on the matrix cores: this package's
                                                (`ep_hip_gemm_bf16`) where it runs blocks of 64 x 64, the vendor library's
                                                otherwise (`TILED_PRODUCT = "auto"`, the default; `"own"` and `"library"`
                                                force one of them)

"fused_through_lds": any M, weight never written. One kernel (`ep_hip_linear_fused_mfma_bf16`) in which every workgroup
decodes 32 tiles whose chains stay aligned in k, passes each group of decoded vectors through an LDS ring and multiplies
them on the matrix cores (`v_mfma_f32_32x32x16_bf16`) with activations it streams from memory; containers it cannot take
(no two-level tables: prob_bits 12 and up, alphabets beyond a byte; rows of an odd number of vectors) fall through to
"fused". It is correct to the same tolerance and slower than "fused" everywhere it was measured (MI355X, kernel times):
3072 x 3072 @ 4 bpp, M = 16 / 256 / 4096: 129 / 184 / 447 us (+ 11-53 us for its two small helper kernels) against 90 /
92 / 130 us for decode + product. The reasons are the format's, not the kernel's: a tile yields 32 vectors per chain of
nine dependent steps whatever is fused behind it, so a workgroup's operand is 32 weight rows wide per 256 k and every
activation byte it loads meets only 32 weight rows (a tiled GEMM reuses it 192-256 times: 2.4 GB of activation traffic
from L2 at M = 4096 where the GEMM needs 0.7 GB); gathering 32 aligned tiles on one compute unit puts four chains on every
SIMD, which lengthens each chain step from 138 to 219 ns; and for M > 256 the same tiles are decoded once per block of
256 activation rows. It stays in the package as the built and measured form of the idea, selected only by name.

Which tiled product, measured on an MI355X with the weight coming from memory, as a weight that has just been decoded
does (3072 x 3072 weight, this package's kernels / the vendor library's): 256 rows 16.9 / 19.4 us, 1024 rows 28.4 / 29.5 us,
4096 rows 67.3 / 63.2 us. A product of few tiles is bounded by the rate at which one compute unit takes operand bytes, and
this package's kernel for it (blocks of 64 x 64, four stages of loads in flight) is the faster one on every layer shape
tried (13-35 %); from there on the two are within 10 % of each other, one ahead here and the other there, and the
default leaves those to the library. The reference has one path for every M: decode, then `F.linear`
(entropack/linear/linear.py:163-165).

The forward is differentiable with respect to the activations (like the reference's `F.linear` on a constant weight):
under autograd the kernels run inside a `torch.autograd.Function` whose backward multiplies the output gradient with
the decoded weight.
"""
import torch
from torch.nn import functional as F

from ..schemes.base import packed_buffers
from ..schemes.lattice_rans import hip as hip_lane
from ..schemes.lattice_rans.format import LatticeBuffers
from . import kernels

#: Which tiled GEMM multiplies more than `kernels.SKINNY_MAX_ROWS` activation rows in fused mode: "auto" (this package's where
#: it runs its blocks of 64 x 64, else the library's), "library" or "own".
TILED_PRODUCT = "auto"


def _forward_kernels(layer, x: torch.Tensor) -> torch.Tensor:
    container = layer._container()
    if container.compress_method == "lattice_rans" and container.encoded_dtype == torch.bfloat16:
        on_device = container.to(device=x.device)
        buffers = packed_buffers(on_device.buffers, LatticeBuffers)
        if layer.forward_mode == "fused_through_lds" and hip_lane.mfma_linear_usable(buffers, tuple(container.shape), x):
            return hip_lane.linear_mfma(buffers, shape=tuple(container.shape), x=x, bias=layer._bias_on(x.device))
        if hip_lane.fused_linear_pays(buffers, tuple(container.shape), x):
            return hip_lane.linear_rows(buffers, shape=tuple(container.shape), x=x, bias=layer._bias_on(x.device))
    weight = layer._decoded_for(x)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("the fused forward runs in bfloat16; use forward_mode='decode_then_gemm' for other dtypes")
    rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
    if rows > kernels.SKINNY_MAX_ROWS and TILED_PRODUCT != "own":
        if TILED_PRODUCT == "library" or not kernels.takes_small_blocks(rows, weight.shape[0], x.shape[-1] * 2, x.device):
            return F.linear(x, weight, layer._bias_on(x.device))
    return kernels.gemm_bf16(x, weight, layer._bias_on(x.device), out_dtype=x.dtype)


class _FusedLinearFunction(torch.autograd.Function):
    """The fused forward with the input gradient of y = x W^T: grad_x = grad_y W, W decoded again in the backward (the
    compressed weight and the bias are frozen and get no gradient)."""

    @staticmethod
    def forward(ctx, x, layer):
        ctx.layer = layer
        ctx.input_shape = tuple(x.shape)
        return _forward_kernels(layer, x.detach())

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        rows = grad_output.reshape(-1, grad_output.shape[-1])
        dense = ctx.layer.dequantize(rows.device).to(rows.dtype)
        return (rows @ dense).reshape(ctx.input_shape), None


def linear_forward(layer, x: torch.Tensor) -> torch.Tensor:
    if torch.is_grad_enabled() and x.requires_grad:
        return _FusedLinearFunction.apply(x, layer)
    return _forward_kernels(layer, x)


def int8_linear_forward(layer, activation: torch.Tensor, activation_scale: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    if layer.forward_mode == "fused_through_lds":
        container = layer._container()
        if container.compress_method == "lattice_rans" and container.encoded_dtype == torch.int8:
            on_device = container.to(device=activation.device)
            buffers = packed_buffers(on_device.buffers, LatticeBuffers)
            if hip_lane.mfma_linear_usable(buffers, tuple(container.shape), activation):
                return hip_lane.linear_mfma_i8(buffers, shape=tuple(container.shape), activation=activation, activation_scale=activation_scale,
                                               weight_scale=layer._scale(activation.device), bias=layer._bias_on(activation.device),
                                               out_dtype=out_dtype)
    codes = layer._decoded_for(activation)
    return kernels.int8_gemm(activation, codes, activation_scale, layer._scale(codes.device), layer._bias_on(activation.device), out_dtype)
