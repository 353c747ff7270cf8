"""Linear layers whose weight lives compressed and is decoded on the MI355X in every forward.

`CompressedLinear` and `CompressedINT8Linear` keep the constructor, `from_linear`, `forward`, `dequantize`,
`compress_weight`, `stored_nbytes`, `compressed_bits` and the `state_dict` layout (`<prefix>weight.entropack_quant_state`,
a 1-D uint8 blob) of the reference layers (entropack/linear/linear.py:18-230, 249-391, 447-490). Differences that
the change of hardware forces:

  * decoding selects the `hip` backend (the reference hard-codes "cuda", linear.py:15,58-68); encoding, which the
    reference also runs on its CUDA lane, runs on this package's device encoder for a weight that is on the GPU and
    on its CPU encoder for a weight that is on the host;
  * `forward` has two modes. "decode_then_gemm" materialises the dense weight with the decode kernel and multiplies
    with the library GEMM, exactly the reference's data flow. "fused" picks by the number of activation rows
    (`linear/fused.py`): for one row (up to four on weights large enough that their decode is bound by throughput) the decode kernel multiplies
    in registers and the dense weight is never written; beyond that the weight is decoded to memory once and
    multiplied by the split-K skinny product (up to 128 rows) or a tiled matrix-core product. "fused_through_lds" is the
    one kernel for any number of rows in which the matrix cores multiply decoded tiles taken from LDS (the weight is
    never written either); it is slower than "fused" on every shape measured and exists as the measured answer to
    "why not fuse decode and GEMM" (`linear/fused.py`);
  * the W8A8 layer gates on a gfx950 device instead of a CUDA compute capability (linear.py:324-336) and its int8
    GEMM + row quantiser are HIP kernels with the semantics of the reference's Triton kernels
    (entropack/linear/quant_kernels.py:15-79).
"""
import dataclasses
from numbers import Real
from typing import ClassVar

import torch
from torch.nn import functional as F

from ..backends import hip as _hip
from ..compression import CompressedTensor, compress, decompress
from ..registry import default_config, get_scheme, name_for_config, require_dtype
from ..schemes import EntroPackLossyConfig, RawConfig
from . import convrot

QUANT_STATE_LEAF = "entropack_quant_state"      # state_dict key suffix of a compressed weight (the reference's, linear.py:190-230)
#: Lane that compresses a weight: the device lane for a weight that is on the GPU (the reference's layers use their
#: device lane for both directions, linear.py:15,59-68), the CPU lane for a weight on the CPU.
ENCODE_BACKEND_BY_DEVICE = {"cuda": "hip", "cpu": "eager"}
DECODE_BACKEND = "hip"
FORWARD_MODES = ("decode_then_gemm", "fused", "fused_through_lds")
_F32_EPS = torch.finfo(torch.float32).eps


class CompressedLinear(torch.nn.Linear):
    """`torch.nn.Linear` with a frozen, compressed weight.

    Args:
        in_features, out_features, bias: as for `torch.nn.Linear`; the bias stays dense.
        config: compression config; None picks a scheme by dtype.
        device: device of the bias; the compressed buffers stay where the source weight was.
        dtype: container dtype the weight is compressed in.
        forward_mode: "decode_then_gemm" (default), "fused", or "fused_through_lds" (see `linear/fused.py`).
    """

    state_buffer_names: ClassVar[tuple[str, ...]] = ()
    state_buffer_dtypes: ClassVar[dict[str, torch.dtype]] = {}

    def __init__(self, in_features: int, out_features: int, bias: bool = True, *, config=None,
                 device: str | torch.device | None = None, dtype: torch.dtype = torch.bfloat16,
                 forward_mode: str = "decode_then_gemm"):
        with torch.device("meta"):
            super().__init__(in_features, out_features, bias=False, dtype=dtype)
        if forward_mode not in FORWARD_MODES:
            raise ValueError(f"forward_mode must be one of {FORWARD_MODES}, got {forward_mode!r}")
        self.forward_mode = forward_mode
        self._decode_ahead = None          # a linear.ahead.DecodeAhead serving this layer's weight, if attached
        self.config = config
        self._init_dtype = require_dtype(dtype)
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(out_features, dtype=dtype, device=device), requires_grad=False)
        if config is not None:
            scheme = get_scheme(name_for_config(config))
            if not scheme.supports(self.container_dtype):
                raise ValueError(f"'{scheme.name}' does not support format {self.container_dtype}")
        self.weight = torch.nn.Parameter(torch.zeros(0, dtype=self._init_dtype, device=device), requires_grad=False)
        for name in self.state_buffer_names:
            self.register_buffer(name, torch.zeros(out_features, dtype=self.state_buffer_dtypes[name], device=device), persistent=True)

    # -- configs --------------------------------------------------------------------------------------------

    def _config_on(self, backend: str):
        if self.config is not None:
            return dataclasses.replace(self.config, execution_backend=backend)
        if isinstance(self.weight, CompressedTensor):
            return self.weight.scheme.make_config({"execution_backend": backend})
        return default_config(self.container_dtype, execution_backend=backend)

    def _encode_config_for(self, tensor: torch.Tensor):
        return self._config_on(ENCODE_BACKEND_BY_DEVICE.get(tensor.device.type, "eager"))

    @property
    def _decode_config(self):
        return self._config_on(DECODE_BACKEND)

    @property
    def container_dtype(self) -> torch.dtype:
        """The dtype the weight was compressed in; layer `.to(dtype)` casts do not change it."""
        return self._init_dtype

    # -- size bookkeeping -------------------------------------------------------------------------------------

    @property
    def qweight(self) -> torch.Tensor:
        """The packed blob, under the name quantisation frameworks look for."""
        return self.weight.entropack_quant_state if isinstance(self.weight, CompressedTensor) else self.bias

    @property
    def stored_nbytes(self) -> int:
        total = self.weight.storage_nbytes()
        for name in self.state_buffer_names:
            extra = self._buffers.get(name)
            if extra is not None:
                total += extra.numel() * extra.element_size()
        return total

    @property
    def compressed_bits(self) -> float:
        rows, cols = self.weight.shape
        return 8 * self.stored_nbytes / (rows * cols)

    # -- compress / decode ------------------------------------------------------------------------------------

    def _check_weight_shape(self, shape) -> None:
        wanted = (self.out_features, self.in_features)
        if tuple(shape) != wanted:
            raise ValueError(f"weight has shape {tuple(shape)}, but the layer expects {wanted}")

    def _compress_tensor(self, tensor: torch.Tensor) -> CompressedTensor:
        packed = compress(tensor.to(self.container_dtype), self._encode_config_for(tensor))
        if packed.compress_method == "raw" and "reason" in packed.header:
            raise RuntimeError(
                f"{packed.header['requested']} cannot store a {tuple(tensor.shape)} {self.container_dtype} weight for "
                f"{type(self).__name__}: {packed.header['reason']}")
        return packed

    def compress_weight(self, weight: torch.Tensor) -> None:
        """Compress `weight` and make it this layer's weight."""
        self._check_weight_shape(weight.shape)
        self.weight = torch.nn.Parameter(self._compress_tensor(weight.detach()), requires_grad=False)

    def _container(self) -> CompressedTensor:
        if not isinstance(self.weight, CompressedTensor):
            raise RuntimeError(
                f"{type(self).__name__}({self.in_features}, {self.out_features}) has nothing to decode: "
                "the weight was not correctly loaded")
        return self.weight

    def _reconstruct(self, device=None) -> torch.Tensor:
        return decompress(self._container().to(device=device), self._decode_config)

    def dequantize(self, device=None) -> torch.Tensor:
        """The dense weight, decoded on `device` (default: where the container lives)."""
        return self._reconstruct(device)

    def _decoded_for(self, x: torch.Tensor) -> torch.Tensor:
        """The container decoded in its own dtype for one product with `x`: from an attached DecodeAhead when autograd
        will not keep the tensor (its memory is reused a few layers on), else decoded here."""
        ahead = self._decode_ahead
        if ahead is not None and x.device == ahead.device and not (torch.is_grad_enabled() and x.requires_grad):
            weight = ahead.weight_of(self)
            if weight is not None:
                return weight
        return decompress(self._container().to(device=x.device), self._decode_config)

    @classmethod
    def from_linear(cls, linear: torch.nn.Linear, **kwargs) -> "CompressedLinear":
        """A layer of this class holding `linear`'s weight compressed and a copy of its bias."""
        weight = linear.weight
        if weight is None or weight.device.type == "meta":
            raise ValueError("cannot compress a Linear whose weight is not materialized")
        kwargs.setdefault("dtype", weight.dtype)
        layer = cls(linear.in_features, linear.out_features, bias=linear.bias is not None, device=weight.device, **kwargs)
        layer.compress_weight(weight.data)
        if linear.bias is not None:
            layer.bias = torch.nn.Parameter(linear.bias.data.clone(), requires_grad=False)
        return layer

    @property
    def device(self) -> torch.device:
        if self.weight is not None:
            return self.weight.device
        return self.bias.device if self.bias is not None else torch.device("meta")

    def _bias_on(self, device) -> torch.Tensor | None:
        return None if self.bias is None else self.bias.to(device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.forward_mode != "decode_then_gemm":
            from . import fused
            return fused.linear_forward(self, x)
        return F.linear(x, self._decoded_for(x).to(x.dtype), self._bias_on(x.device))

    def extra_repr(self) -> str:
        scheme = "auto" if self.config is None else name_for_config(self.config)
        parts = [f"scheme={scheme}", f"container={str(self.container_dtype).split('.', 1)[1]}", f"mode={self.forward_mode}"]
        if isinstance(self.weight, CompressedTensor):
            parts.append(f"bits={self.compressed_bits:.3f}")
        return ", ".join(parts)

    # -- module plumbing --------------------------------------------------------------------------------------

    def _apply(self, fn, recurse=True):
        # Module.to(dtype) must not cast the float32 row scales of the W8A8 layers.
        parked = {name: self._buffers.pop(name) for name in self.state_buffer_names if name in self._buffers}
        try:
            super()._apply(fn, recurse=recurse)
        finally:
            for name, tensor in parked.items():
                if tensor is None:
                    self._buffers[name] = None
                else:
                    moved = fn(tensor)
                    self._buffers[name] = moved if moved.dtype == tensor.dtype else tensor.to(device=moved.device)
        return self

    def _save_to_state_dict(self, destination: dict, prefix: str, keep_vars: bool) -> None:
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if isinstance(self.weight, CompressedTensor):
            # the wrapper tensor has no storage a checkpoint could hold; the packed blob stands in for it
            del destination[prefix + "weight"]
            blob = getattr(self.weight, QUANT_STATE_LEAF)
            destination[prefix + "weight." + QUANT_STATE_LEAF] = blob if keep_vars else blob.detach()

    def _home_for(self, blob: torch.Tensor) -> torch.device:
        """Where a loaded blob should live: with the weight it replaces, else with the bias, else where it is."""
        for holder in (self._parameters.get("weight"), self.bias):
            if holder is not None and holder.device.type != "meta":
                return holder.device
        return blob.device

    def _adopt_blob(self, blob: torch.Tensor, in_place: bool) -> None:
        """Make the container packed in `blob` this layer's weight. `in_place`: keep the existing Parameter object alive
        (optimisers and hooks hold on to it) and keep its device."""
        # Unpacked where the blob is (a checkpoint's is on the host: the header is read there) and moved as a container,
        # which takes host copies of the small tables along for the decode plan.
        container = CompressedTensor.unpack(blob)
        if in_place:
            home = self._home_for(blob)
            container = container.to(device=home, copy=True) if home != blob.device else container.clone()
        self._check_weight_shape(container.shape)
        fresh = torch.nn.Parameter(container, requires_grad=False)
        present = self._parameters.get("weight")
        if in_place and isinstance(present, CompressedTensor):
            torch.utils.swap_tensors(present, fresh)
        else:
            self._parameters["weight"] = fresh

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        entry = prefix + "weight." + QUANT_STATE_LEAF
        blob = state_dict.pop(entry, None)
        if blob is None:
            if strict:
                missing_keys.append(entry)
        else:
            try:
                self._adopt_blob(blob, in_place=not local_metadata.get("assign_to_params_buffers", False))
            except (TypeError, ValueError) as problem:
                error_msgs.append(f"{prefix[:-1]}: {problem}")
        # nn.Module must neither look for a dense "weight" entry nor report the blob's key as unexpected
        held = self._parameters.pop("weight")
        try:
            super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)
        finally:
            self._parameters["weight"] = held


class _W8A8Function(torch.autograd.Function):
    """8-bit forward with a straight-through input gradient: d(out)/d(x) is taken through the dequantised weight, the
    compressed weight itself gets no gradient."""

    @staticmethod
    def forward(ctx, x, layer):
        ctx.layer = layer
        ctx.input_shape = tuple(x.shape)
        return layer._forward8(x.detach())

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        rows = grad_output.reshape(-1, grad_output.shape[-1])
        dense = ctx.layer.dequantize(rows.device).to(rows.dtype)
        return (rows @ dense).reshape(ctx.input_shape), None


class QuantizedLinear(CompressedLinear):
    """W8A8 base: the weight is quantised per row to 8-bit codes (scale kept in `weight_quant_scale`), the codes are
    stored raw or lattice-coded, and activations are quantised per row at run time."""

    code_dtype: ClassVar[torch.dtype]
    code_max: ClassVar[float]
    rounds_to_integer: ClassVar[bool]
    state_buffer_names = ("weight_quant_scale",)
    state_buffer_dtypes = {"weight_quant_scale": torch.float32}

    def __init__(self, in_features: int, out_features: int, bias: bool = True, *, config=None, device=None,
                 dtype: torch.dtype = torch.bfloat16, forward_mode: str = "decode_then_gemm"):
        super().__init__(in_features, out_features, bias=bias, config=self._coded(config), device=device, dtype=dtype,
                         forward_mode=forward_mode)

    @property
    def container_dtype(self) -> torch.dtype:
        return self.code_dtype

    @classmethod
    def _coded(cls, config):
        """The config the codes are stored with: raw by default, or lattice-coded below the codes' own 8 bits."""
        if config is None or isinstance(config, RawConfig):
            return config or RawConfig()
        if isinstance(config, EntroPackLossyConfig):
            rate = config.target_bpp
            usable = isinstance(rate, Real) and not isinstance(rate, bool) and 0.0 < float(rate) < 8.0
            if not usable:
                raise ValueError(f"{cls.__name__} stores {cls.code_dtype} codes, 8 bits wide, so a target_bpp only pays below 8; "
                                 f"got {rate!r}. Pass RawConfig to store the codes uncoded.")
            return config
        raise TypeError(f"{cls.__name__} stores {cls.code_dtype} codes: either uncoded (RawConfig) or lattice-coded "
                        f"(EntroPackLossyConfig), got {type(config).__name__}")

    def _quantize_rows(self, tensor: torch.Tensor):
        """Per-row absmax quantisation in plain torch (used for the weight, once, on any device)."""
        flat = tensor.reshape(-1, tensor.shape[-1]).float()
        scale = (flat.abs().amax(dim=1) / self.code_max).clamp(min=_F32_EPS)
        scaled = flat / scale.unsqueeze(1)
        if self.rounds_to_integer:
            scaled = scaled.round()
        return scaled.clamp(-self.code_max, self.code_max).to(self.code_dtype), scale

    def compress_weight(self, weight: torch.Tensor) -> None:
        self._check_weight_shape(weight.shape)
        codes, scale = self._quantize_rows(self._prepare_weight_source(weight.detach()))
        self.weight = torch.nn.Parameter(self._compress_tensor(codes), requires_grad=False)
        self.weight_quant_scale = scale

    def _prepare_weight_source(self, weight: torch.Tensor) -> torch.Tensor:
        """The basis the codes are taken in (the identity here)."""
        return weight

    def _restore_weight_basis(self, weight: torch.Tensor) -> torch.Tensor:
        return weight

    def codes(self, device=None) -> torch.Tensor:
        """The weight codes in `code_dtype`, decoded on `device`."""
        return decompress(self._container().to(device=device, dtype=self.code_dtype), self._decode_config)

    def _scale(self, device) -> torch.Tensor:
        return self.weight_quant_scale.to(device=device, dtype=torch.float32)

    def dequantize(self, device=None) -> torch.Tensor:
        codes = self.codes(device)
        return self._restore_weight_basis(codes.float() * self._scale(codes.device).unsqueeze(1)).to(self._init_dtype)

    def _require_8bit_gemm(self, device: torch.device) -> None:
        reason = _hip.probe() if device.type == "cuda" else f"tensor is on {device}"
        if reason is not None:
            raise RuntimeError(f"{type(self).__name__} needs an MI355X (gfx950) device for its 8-bit matrix cores: {reason}")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        self._require_8bit_gemm(x.device)
        if x.requires_grad:
            return _W8A8Function.apply(x, self)
        return self._forward8(x)

    def _forward8(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class CompressedINT8Linear(QuantizedLinear):
    """Symmetric int8 weights and activations: y = (A_i8 . W_i8^T)_i32 * sa[m] * sw[n] + b[n], cast to x.dtype.

    `use_convrot=True` rotates groups of `convrot_groupsize` input features (a power of four, lowered by factors of four
    until it divides `in_features`) of the weight before it is quantised and of the activations before they are: the
    product is unchanged, outliers are spread. Like the reference (entropack/linear/linear.py:445-478) the flag is a
    constructor argument, not part of the checkpoint.
    """

    code_dtype = torch.int8
    code_max = 127.0
    rounds_to_integer = True

    def __init__(self, in_features: int, out_features: int, bias: bool = True, *, config=None, device=None,
                 dtype: torch.dtype = torch.bfloat16, forward_mode: str = "decode_then_gemm", use_convrot: bool = False,
                 convrot_groupsize: int = 256):
        self.use_convrot = bool(use_convrot)
        self._convrot_group = convrot.choose_convrot_group(in_features, convrot_groupsize) if self.use_convrot else None
        if self.use_convrot and self._convrot_group is None:
            raise ValueError(f"use_convrot requires in_features {in_features} to contain a power-of-four group; "
                             f"got convrot_groupsize={convrot_groupsize}")
        super().__init__(in_features, out_features, bias=bias, config=config, device=device, dtype=dtype, forward_mode=forward_mode)

    def _rotation(self, like: torch.Tensor) -> torch.Tensor:
        return convrot.build_convrot_matrix(self._convrot_group, device=like.device, dtype=like.dtype)

    def _prepare_weight_source(self, weight: torch.Tensor) -> torch.Tensor:
        if not self.use_convrot:
            return weight
        return convrot.rotate_weight(weight, self._rotation(weight), self._convrot_group)

    def _restore_weight_basis(self, weight: torch.Tensor) -> torch.Tensor:
        if not self.use_convrot:
            return weight
        return convrot.rotate_weight(weight, self._rotation(weight), self._convrot_group, inverse=True)

    def _forward8(self, x: torch.Tensor) -> torch.Tensor:
        from . import kernels
        flat = x.reshape(-1, x.shape[-1]).contiguous()
        if self.use_convrot:
            activation, activation_scale = kernels.rotate_quantize_rows(flat.detach(), self._convrot_group)
        else:
            activation, activation_scale = kernels.quantize_rows(flat.detach())
        if self.forward_mode != "decode_then_gemm":
            from . import fused
            out = fused.int8_linear_forward(self, activation, activation_scale, x.dtype)
        else:
            codes = self._decoded_for(flat.detach())
            out = kernels.int8_gemm(activation, codes, activation_scale, self._scale(codes.device), self._bias_on(x.device), x.dtype)
        return out.reshape(*x.shape[:-1], self.out_features)


__all__ = ["CompressedINT8Linear", "CompressedLinear", "QuantizedLinear"]
