"""Block rotation of W8A8 layers: the matrix, the group choice and the weight side (CPU); the fused activation kernel
and the layer forward are checked on the GPU in test_hip_linear.py.

The definition is the reference's (entropack/linear/convrot.py:9-53): Kronecker powers of the 4 x 4 seed below over
sqrt(order). Nothing here evaluates the package's own construction (digit complements of i ^ j) to get the expectation.
"""
import math

import pytest
import torch

import entropack_amd as ep
from entropack_amd.linear import convrot

SEED = torch.tensor([[1.0, 1.0, 1.0, -1.0], [1.0, 1.0, -1.0, 1.0], [1.0, -1.0, 1.0, 1.0], [-1.0, 1.0, 1.0, 1.0]])


def kron_power(order):
    matrix = SEED
    while matrix.shape[0] < order:
        matrix = torch.kron(matrix, SEED)
    return matrix / math.sqrt(order)


@pytest.mark.parametrize("order", [4, 16, 64, 256, 1024])
def test_matrix_is_the_kronecker_power_symmetric_and_its_own_inverse(order):
    matrix = convrot.build_convrot_matrix(order, device="cpu", dtype=torch.float32)
    assert torch.equal(matrix, kron_power(order))
    assert torch.equal(matrix, matrix.t())
    assert torch.allclose(matrix @ matrix, torch.eye(order), atol=1e-6)
    assert convrot.build_convrot_matrix(order, device="cpu", dtype=torch.float32) is matrix          # cached
    assert convrot.build_convrot_matrix(order, device="cpu", dtype=torch.bfloat16).dtype == torch.bfloat16


def test_group_rules():
    assert [v for v in range(1, 5000) if convrot.is_convrot_group(v)] == [4, 16, 64, 256, 1024, 4096]
    assert not convrot.is_convrot_group(True) and not convrot.is_convrot_group(16.0) and not convrot.is_convrot_group("16")
    assert convrot.choose_convrot_group(3072) == 256 and convrot.choose_convrot_group(3072, 1024) == 1024
    assert convrot.choose_convrot_group(3136) == 64 and convrot.choose_convrot_group(100) == 4
    assert convrot.choose_convrot_group(50) is None and convrot.choose_convrot_group(4096, 16) == 16
    for bad in (0, 8, 32, 100, 2.0):
        with pytest.raises(ValueError, match="power of four"):
            convrot.choose_convrot_group(256, bad)
    with pytest.raises(ValueError, match="power of four"):
        convrot.build_convrot_matrix(8, device="cpu", dtype=torch.float32)


def test_rotations_act_group_by_group_and_undo_each_other():
    torch.manual_seed(0)
    weight = torch.randn(6, 192, dtype=torch.float64)
    matrix = convrot.build_convrot_matrix(64, device="cpu", dtype=torch.float64)
    turned = convrot.rotate_weight(weight, matrix, 64)
    for g in range(3):
        assert torch.allclose(turned[:, 64 * g:64 * (g + 1)], weight[:, 64 * g:64 * (g + 1)] @ kron_power(64).double().t(), atol=1e-12)
    assert torch.allclose(convrot.rotate_weight(turned, matrix, 64, inverse=True), weight, atol=1e-12)
    x = torch.randn(2, 5, 192, dtype=torch.float64)
    rotated = convrot.rotate_activation(x, matrix, 64)
    assert rotated.shape == x.shape
    assert torch.allclose(rotated @ turned.t(), x @ weight.t(), atol=1e-10)          # the product is unchanged
    with pytest.raises(ValueError, match="not divisible"):
        convrot.rotate_activation(torch.zeros(3, 100), matrix, 64)
    with pytest.raises(ValueError):
        convrot.rotate_weight(torch.zeros(2, 3, 64), matrix, 64)


def test_int8_layer_takes_its_codes_in_the_rotated_basis():
    torch.manual_seed(1)
    dense = torch.nn.Linear(320, 24, dtype=torch.float32)
    dense.weight.data[:, 7] *= 30.0                                    # an outlier input channel
    plain = ep.CompressedINT8Linear.from_linear(dense)
    turned = ep.CompressedINT8Linear.from_linear(dense, use_convrot=True)
    assert turned.use_convrot and turned._convrot_group == 64 and not plain.use_convrot
    assert ep.CompressedINT8Linear.from_linear(dense, use_convrot=True, convrot_groupsize=16)._convrot_group == 16
    rotated = dense.weight.data.reshape(24, 5, 64) @ kron_power(64).t()
    scale = (rotated.reshape(24, 320).abs().amax(dim=1) / 127.0).clamp(min=torch.finfo(torch.float32).eps)
    assert torch.equal(turned.weight_quant_scale, scale)
    assert torch.equal(turned.codes("cpu"), (rotated.reshape(24, 320) / scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8))
    # dequantize undoes the rotation, and spreading the outlier lowers the weight error
    error_turned = (turned.dequantize() - dense.weight.data).norm()
    error_plain = (plain.dequantize() - dense.weight.data).norm()
    assert error_turned < 0.5 * error_plain
    assert set(turned.state_dict()) == set(plain.state_dict())                     # the flag is not part of the checkpoint
    with pytest.raises(ValueError, match="power-of-four group"):
        ep.CompressedINT8Linear(50, 8, use_convrot=True)
    with pytest.raises(ValueError, match="power of four"):
        ep.CompressedINT8Linear(64, 8, use_convrot=True, convrot_groupsize=32)
