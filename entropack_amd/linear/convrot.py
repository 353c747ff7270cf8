"""Block rotation for W8A8 layers ("ConvRot"): weights are rotated once before they are quantised, activations on
every forward before theirs, so that outliers are spread over a group of input features.

Same definitions as the reference (entropack/linear/convrot.py:9-61): groups of `g = 4**k` consecutive input features
are multiplied with R_g = kron^k(S) / 2**k, S = ones(4, 4) - 2 * antidiagonal. S is symmetric with S @ S = 4 I, so R_g is
symmetric and its own inverse; entry (i, j) of kron^k(S) is -1 for every base-4 digit position in which i and j are
complements (digit_i + digit_j = 3, i.e. both bits of i ^ j set) and +1 otherwise, which is how the matrix is built
here. The device-side rotation of activations is fused into the row quantiser (ep_hip_rotate_quantize_rows).
"""
import torch

#: Largest group the fused rotate-and-quantise kernel handles; larger groups rotate through a library product.
FUSED_GROUP_LIMIT = 256

_matrices: dict[tuple, torch.Tensor] = {}


def is_convrot_group(value: object) -> bool:
    """True for 4, 16, 64, 256, ... given as a plain int."""
    if type(value) is not int or value < 4:
        return False
    return value & (value - 1) == 0 and value.bit_length() % 2 == 1


def choose_convrot_group(in_features: int, requested: int = 256) -> int | None:
    """The largest power of four not above `requested` that divides `in_features`, or None."""
    if not is_convrot_group(requested):
        raise ValueError(f"convrot group size must be a power of four at least 4, got {requested}")
    size = requested
    while size >= 4:
        if in_features % size == 0:
            return size
        size //= 4
    return None


def build_convrot_matrix(order: int, *, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
    if not is_convrot_group(order):
        raise ValueError(f"convrot order must be a power of four at least 4, got {order}")
    device = torch.device(device)
    key = (order, device.type, device.index, dtype)
    cached = _matrices.get(key)
    if cached is None:
        index = torch.arange(order, dtype=torch.int64)
        differ = index.unsqueeze(1) ^ index.unsqueeze(0)
        both = differ & (differ >> 1) & 0x5555555555555555           # one bit per base-4 digit whose two bits both differ
        flips = torch.zeros_like(both)
        for digit in range(0, order.bit_length(), 2):
            flips += (both >> digit) & 1
        signs = 1.0 - 2.0 * (flips & 1).to(torch.float32)
        cached = (signs / float(1 << ((order.bit_length() - 1) // 2))).to(device=device, dtype=dtype)
        _matrices[key] = cached
    return cached


def _by_groups(rows: torch.Tensor, matrix: torch.Tensor, group: int) -> torch.Tensor:
    features = rows.shape[-1]
    if features % group:
        raise ValueError(f"in_features {features} is not divisible by convrot group {group}")
    blocks = rows.reshape(-1, features // group, group)
    return torch.matmul(blocks, matrix.to(blocks.dtype)).reshape(rows.shape)


def rotate_activation(x: torch.Tensor, matrix: torch.Tensor, group: int) -> torch.Tensor:
    """x[..., K] with every group of K multiplied by `matrix`, in x's dtype (a library product on x's device)."""
    return _by_groups(x, matrix, group)


def rotate_weight(weight: torch.Tensor, matrix: torch.Tensor, group: int, *, inverse: bool = False) -> torch.Tensor:
    """W[N, K] -> W with every group of K multiplied by matrix^T (or by matrix, to undo it)."""
    if weight.dim() != 2:
        raise ValueError(f"rotate_weight takes a [out_features, in_features] matrix, got {tuple(weight.shape)}")
    return _by_groups(weight, matrix if inverse else matrix.t(), group)


__all__ = ["build_convrot_matrix", "choose_convrot_group", "is_convrot_group", "rotate_activation", "rotate_weight"]
