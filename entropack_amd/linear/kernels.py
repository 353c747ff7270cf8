"""Python face of the HIP linear kernels (libentropack_hip.so): MFMA GEMMs and the activation row quantiser.

Same call shapes as the reference's Triton wrappers (entropack/linear/quant_kernels.py:81-106). Everything runs on the
tensors' device and torch's current stream; nothing here has a CPU or library fallback.
"""
import torch

from ..backends import hip as _hip


#: Up to this many activation rows the product is bound by the weight stream and takes the split-K kernel.
SKINNY_MAX_ROWS = 128


def _require_device(*tensors: torch.Tensor) -> torch.device:
    device = tensors[0].device
    if device.type != "cuda":
        raise RuntimeError(f"the HIP linear kernels need device tensors, got {device}")
    for tensor in tensors:
        if tensor is not None and tensor.device != device:
            raise ValueError("all operands must be on one device")
    return device


def _rows(tensor: torch.Tensor) -> torch.Tensor:
    """2-D view with unit inner stride (copying only if the layout forces it)."""
    flat = tensor.reshape(-1, tensor.shape[-1])
    return flat if flat.stride(-1) == 1 and flat.data_ptr() % 16 == 0 and flat.stride(0) % 16 == 0 else flat.contiguous()


def takes_small_blocks(rows: int, outer: int, row_bytes: int, device: torch.device) -> bool:
    """Whether this package's tiled product runs `rows` x `outer` with rows of `row_bytes` bytes of K in blocks of 64 x 64: the
    products on which it is ahead of the vendor library's (host-side rule of the C library)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return bool(_hip.library().ep_hip_gemm_takes_small_blocks(rows, outer, row_bytes, _hip.device_info(index).compute_units))


def gemm_bf16(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x[..., K] @ weight[N, K].T (+ bias): bf16 operands, f32 accumulation on the matrix cores."""
    device = _require_device(x, weight)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("gemm_bf16 takes bfloat16 operands")
    out_dtype = out_dtype or x.dtype
    flat, w = _rows(x), _rows(weight)
    if w.shape[1] != flat.shape[1]:
        raise ValueError(f"inner sizes differ: {flat.shape[1]} vs {w.shape[1]}")
    rows, inner, outer = flat.shape[0], flat.shape[1], w.shape[0]
    out = torch.empty(rows, outer, dtype=out_dtype, device=device)
    if rows == 0:
        return out.reshape(*x.shape[:-1], outer)
    bias_ready = None if bias is None else bias.to(device=device, dtype=out_dtype).contiguous()
    with torch.cuda.device(device):
        lib = _hip.library()
        cus = _hip.device_info(device.index if device.index is not None else torch.cuda.current_device()).compute_units
        split_bytes = lib.ep_hip_gemm_skinny_workspace(rows, outer, inner * 2, cus)      # 0: not a product for the K-split kernels
    if rows <= SKINNY_MAX_ROWS or split_bytes:
        with torch.cuda.device(device):
            workspace = torch.empty(split_bytes, dtype=torch.uint8, device=device)
            _hip.check("ep_hip_gemm_bf16_skinny", lib.ep_hip_gemm_bf16_skinny(
                flat.data_ptr(), w.data_ptr(), None if bias_ready is None else bias_ready.data_ptr(), out.data_ptr(),
                rows, outer, inner, flat.stride(0), w.stride(0), out.stride(0), _hip.FLOAT_KINDS[out_dtype], cus,
                workspace.data_ptr(), workspace.numel(), _hip.current_stream(device)))
        return out.reshape(*x.shape[:-1], outer)
    with torch.cuda.device(device):
        _hip.check("ep_hip_gemm_bf16", _hip.library().ep_hip_gemm_bf16(
            flat.data_ptr(), w.data_ptr(), None if bias_ready is None else bias_ready.data_ptr(), out.data_ptr(),
            rows, outer, inner, flat.stride(0), w.stride(0), out.stride(0), _hip.FLOAT_KINDS[out_dtype],
            _hip.current_stream(device)))
    return out.reshape(*x.shape[:-1], outer)


def quantize_rows(tensor: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-row symmetric int8 codes and float32 scales of a [rows, K] activation."""
    device = _require_device(tensor)
    if tensor.dtype not in _hip.FLOAT_KINDS:
        raise TypeError(f"quantize_rows takes bf16/f16/f32 activations, got {tensor.dtype}")
    flat = tensor.reshape(-1, tensor.shape[-1])
    if flat.stride(-1) != 1:
        flat = flat.contiguous()
    rows, inner = flat.shape
    codes = torch.empty(rows, inner, dtype=torch.int8, device=device)
    scale = torch.empty(rows, dtype=torch.float32, device=device)
    if rows:
        with torch.cuda.device(device):
            _hip.check("ep_hip_quantize_rows", _hip.library().ep_hip_quantize_rows(
                flat.data_ptr(), _hip.FLOAT_KINDS[tensor.dtype], rows, inner, flat.stride(0), codes.data_ptr(),
                scale.data_ptr(), _hip.current_stream(device)))
    return codes, scale


def rotate_quantize_rows(tensor: torch.Tensor, group: int) -> tuple[torch.Tensor, torch.Tensor]:
    """`quantize_rows` of the block-rotated activation (groups of `group` features, see `linear.convrot`).

    Groups up to 256 rotate inside the quantiser kernel; larger ones (and rows the kernel's 8/16-byte loads cannot take)
    rotate through a library product on the same device first.
    """
    from . import convrot
    device = _require_device(tensor)
    if tensor.dtype not in _hip.FLOAT_KINDS:
        raise TypeError(f"rotate_quantize_rows takes bf16/f16/f32 activations, got {tensor.dtype}")
    flat = tensor.reshape(-1, tensor.shape[-1])
    if flat.stride(-1) != 1:
        flat = flat.contiguous()
    rows, inner = flat.shape
    if not convrot.is_convrot_group(group) or inner % group:
        raise ValueError(f"convrot group {group} must be a power of four dividing in_features {inner}")
    if rows and group <= convrot.FUSED_GROUP_LIMIT:
        codes = torch.empty(rows, inner, dtype=torch.int8, device=device)
        scale = torch.empty(rows, dtype=torch.float32, device=device)
        with torch.cuda.device(device):
            status = _hip.library().ep_hip_rotate_quantize_rows(
                flat.data_ptr(), _hip.FLOAT_KINDS[tensor.dtype], rows, inner, flat.stride(0), group, codes.data_ptr(),
                scale.data_ptr(), _hip.current_stream(device))
        if status == _hip.OK:
            return codes, scale
        if status != _hip.EUNSUPPORTED:
            _hip.check("ep_hip_rotate_quantize_rows", status)
    matrix = convrot.build_convrot_matrix(group, device=device, dtype=flat.dtype)
    return quantize_rows(convrot.rotate_activation(flat, matrix, group))


def int8_gemm(activation: torch.Tensor, codes: torch.Tensor, activation_scale: torch.Tensor, weight_scale: torch.Tensor,
              bias: torch.Tensor | None, out_dtype: torch.dtype) -> torch.Tensor:
    """(activation[M, K] @ codes[N, K].T) in int32, times both row scales, plus bias, as `out_dtype`."""
    device = _require_device(activation, codes, activation_scale, weight_scale)
    if activation.dtype != torch.int8 or codes.dtype != torch.int8:
        raise TypeError("int8_gemm takes int8 operands")
    rows, inner = activation.shape
    outer = codes.shape[0]
    if codes.shape[1] != inner:
        raise ValueError(f"inner sizes differ: {inner} vs {codes.shape[1]}")
    a, b = activation, codes
    if inner % 16:                                   # the int8 matrix-core step is 32 wide; rows must be 16-byte multiples
        pad = 16 - inner % 16
        a = torch.nn.functional.pad(a, (0, pad))
        b = torch.nn.functional.pad(b, (0, pad))
    a, b = _rows(a), _rows(b)
    out = torch.empty(rows, outer, dtype=out_dtype, device=device)
    if rows == 0:
        return out
    bias_ready = None if bias is None else bias.to(device=device, dtype=out_dtype).contiguous()
    scale_a, scale_b = activation_scale.float().contiguous(), weight_scale.float().contiguous()
    with torch.cuda.device(device):
        lib = _hip.library()
        cus = _hip.device_info(device.index if device.index is not None else torch.cuda.current_device()).compute_units
        split_bytes = lib.ep_hip_gemm_skinny_workspace(rows, outer, a.shape[1], cus)     # 0: not a product for the K-split kernels
    if rows <= SKINNY_MAX_ROWS or split_bytes:
        with torch.cuda.device(device):
            workspace = torch.empty(split_bytes, dtype=torch.uint8, device=device)
            _hip.check("ep_hip_gemm_i8_skinny", lib.ep_hip_gemm_i8_skinny(
                a.data_ptr(), b.data_ptr(), scale_a.data_ptr(), scale_b.data_ptr(), None if bias_ready is None else bias_ready.data_ptr(),
                out.data_ptr(), rows, outer, a.shape[1], a.stride(0), b.stride(0), out.stride(0), _hip.FLOAT_KINDS[out_dtype], cus,
                workspace.data_ptr(), workspace.numel(), _hip.current_stream(device)))
        return out
    with torch.cuda.device(device):
        _hip.check("ep_hip_gemm_i8", _hip.library().ep_hip_gemm_i8(
            a.data_ptr(), b.data_ptr(), scale_a.data_ptr(), scale_b.data_ptr(), None if bias_ready is None else bias_ready.data_ptr(),
            out.data_ptr(), rows, outer, a.shape[1], a.stride(0), b.stride(0), out.stride(0),
            _hip.FLOAT_KINDS[out_dtype], _hip.current_stream(device)))
    return out
