"""Decode-to-GEMM through LDS (`ep_hip_fused_plan`, `ep_hip_linear_fused_mfma_bf16`): the matrix cores multiply decoded
tiles taken from LDS, the dense weight is never written.

Oracle: y = F.linear(x, decode(W), b) (entropack/linear/linear.py:163-165 of the reference) with W decoded by the CPU
oracle from the same container, in float64, rounded once to bf16; tolerance rel-L2 <= 1e-3 (accumulation order), and no
element further than a few bf16 steps from the float64 value (a dropped or doubled partial sum would be).
"""
import ctypes

import numpy as np
import pytest
import torch
from torch.nn import functional as F

import entropack_amd as ep
from entropack_amd.backends import hip as hip_backend
from entropack_amd.schemes.base import packed_buffers
from entropack_amd.schemes.lattice_rans.format import LatticeBuffers

REL_L2 = 1e-3


def _plan(rows, cols, tile_elements):
    library = hip_backend.library()
    count = ctypes.c_int(0)
    status = library.ep_hip_fused_plan(rows, cols, tile_elements, None, 0, ctypes.byref(count))
    if status != hip_backend.OK:
        return status, None
    batches = (hip_backend.FusedBatch * count.value)()
    assert library.ep_hip_fused_plan(rows, cols, tile_elements, batches, count.value, ctypes.byref(count)) == hip_backend.OK
    return hip_backend.OK, batches


@pytest.mark.parametrize("rows,cols,tile_elements", [
    (3072, 3072, 16384), (3072, 3072, 4096), (8192, 28672, 16384), (3840, 10240, 8192), (64, 288, 288), (1, 256, 16384), (300, 4128, 4100),
])
def test_fused_plan_covers_every_tile_once_with_aligned_chains(rows, cols, tile_elements):
    status, batches = _plan(rows, cols, tile_elements)
    assert status == hip_backend.OK
    vectors_per_row = cols // 8
    tile_vectors = max(32, tile_elements // 9)
    tiles = -(-rows * vectors_per_row // tile_vectors)
    seen = []
    for batch in batches:
        assert batch.base % 4 == 0 and 0 <= batch.base < vectors_per_row
        used = [slot for slot in range(hip_backend.FUSED_SLOTS) if batch.tile[slot] >= 0]
        assert used and used == list(range(len(used)))                   # used slots come first
        for slot in used:
            position = batch.tile[slot] * tile_vectors % vectors_per_row
            assert batch.delta[slot] == position - batch.base and 0 <= batch.delta[slot] <= 31
            seen.append(batch.tile[slot])
    assert sorted(seen) == list(range(tiles))


def test_fused_plan_refuses_rows_it_cannot_align():
    assert _plan(64, 264, 16384)[0] == hip_backend.EUNSUPPORTED            # 33 vectors per row: odd
    assert _plan(64, 272, 16384)[0] == hip_backend.EUNSUPPORTED            # 34 vectors per row: no multiple of four
    assert _plan(64, 128, 16384)[0] == hip_backend.EUNSUPPORTED            # 16 vectors per row: shorter than a group
    assert _plan(0, 256, 16384)[0] == hip_backend.EINVAL
    count = ctypes.c_int(0)
    assert hip_backend.library().ep_hip_fused_plan(64, 256, 16384, None, 0, None) == hip_backend.EINVAL
    one = (hip_backend.FusedBatch * 1)()
    assert hip_backend.library().ep_hip_fused_plan(3072, 3072, 16384, one, 1, ctypes.byref(count)) == hip_backend.EINVAL     # too few


def _host_arrays(container):
    host = {}
    for key, value in container.buffers.items():
        value = value.cpu()
        if value.dtype == torch.uint16:
            host[key] = value.view(torch.int16).numpy().view(np.uint16)
        elif value.dtype == torch.uint32:
            host[key] = value.view(torch.int32).numpy().view(np.uint32)
        else:
            host[key] = value.numpy()
    return host


def _oracle_weight(container):
    from oracle import c_oracle
    rows = container.shape[0]
    cols_padded = int(container.buffers["layout"][0])
    bits = c_oracle.decode(_host_arrays(container), (rows, cols_padded), "bfloat16", threads=8)
    return torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)


def _check(y, x, weight, bias, label):
    exact = F.linear(x.double(), weight.double(), None if bias is None else bias.double())
    expect = exact.float().to(torch.bfloat16).double()
    error = ((y.double() - expect).norm() / expect.norm().clamp_min(1e-30)).item()
    assert error <= REL_L2, (label, error)
    # element by element: within a few bf16 steps of the float64 value, measured on the scale of the row's sum of magnitudes
    scale = F.linear(x.double().abs(), weight.double().abs()) + (0 if bias is None else bias.double().abs())
    assert bool(((y.double() - exact).abs() <= 2.0 ** -7 * exact.abs() + 1e-5 * scale + 1e-30).all()), label


CASES = [
    # rows, cols, bpp, tile_elements (None = default), activation rows
    (3072, 3072, 4.0, None, (1, 5, 33, 100, 256, 300)),
    (512, 1024, 4.0, 4096, (7, 64)),
    (256, 288, 3.5, 288, (3, 40)),              # 36 vectors per row, tiles of 32 vectors: a row boundary in almost every window
    (1000, 2048, 2.0, None, (16, 129)),         # tiles of 3640 vectors, a short last tile
    (130, 4128, 6.0, 4100, (2, 96)),            # 516 vectors per row, odd tile length (455 vectors)
]


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,bpp,tile_elements,activation_rows", CASES)
def test_linear_mfma_matches_f_linear_on_the_oracle_weight(rows, cols, bpp, tile_elements, activation_rows):
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    torch.manual_seed(rows + cols)
    weight = (torch.randn(rows, cols) * 0.02).to(torch.bfloat16)
    weight[rows // 2] = 0                                            # a row of zeros: scale 0 takes the literal formula
    options = {} if tile_elements is None else {"tile_elements": tile_elements}
    container = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager", **options))
    oracle = _oracle_weight(container)[:, :cols].cuda()
    on_gpu = container.to("cuda")
    buffers = packed_buffers(on_gpu.buffers, LatticeBuffers)
    bias = (torch.randn(rows) * 0.01).to(torch.bfloat16).cuda()
    for m in activation_rows:
        print("case fused mfma", (rows, cols, bpp, tile_elements), "M =", m, flush=True)
        x = torch.randn(m, cols).to(torch.bfloat16).cuda()
        assert hip_lane.mfma_linear_usable(buffers, (rows, cols), x)
        for with_bias in (None, bias):
            y = hip_lane.linear_mfma(buffers, shape=(rows, cols), x=x, bias=with_bias)
            torch.cuda.synchronize()
            assert y.shape == (m, rows) and y.dtype == torch.bfloat16
            _check(y, x, oracle, with_bias, (rows, cols, bpp, m, with_bias is not None))
    hip_lane.check_errors(buffers)


@pytest.mark.gpu
def test_linear_mfma_on_randomly_drawn_containers():
    """24 containers from a fixed seed: rows 1..700, 32..640 vectors per row (multiples of four), rates 1.5..7 bpp, tile sizes
    from one group to the default, outlier rows, 1..200 activation rows; every draw against the float64 product on the CPU
    oracle's weight."""
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    rng = np.random.default_rng(20240611)
    done = 0
    while done < 24:
        rows = int(rng.integers(1, 701))
        cols = 8 * 4 * int(rng.integers(8, 161))
        bpp = float(rng.choice([1.5, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0]))
        tile_elements = [None, 288, 300, 1000, 2304, 4096, 4100, 8192][int(rng.integers(0, 8))]
        m = int(rng.integers(1, 201))
        torch.manual_seed(int(rng.integers(0, 1 << 30)))
        weight = torch.randn(rows, cols) * 0.02
        if rng.random() < 0.3:
            weight[int(rng.integers(0, rows))] *= 30.0
        weight = weight.to(torch.bfloat16)
        options = {} if tile_elements is None else {"tile_elements": tile_elements}
        container = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager", **options))
        on_gpu = container.to("cuda")
        buffers = packed_buffers(on_gpu.buffers, LatticeBuffers)
        x = torch.randn(m, cols).to(torch.bfloat16).cuda()
        if not hip_lane.mfma_linear_usable(buffers, (rows, cols), x):      # e.g. a rate whose tables are not the two-level form
            continue
        print("draw", done, (rows, cols, bpp, tile_elements), "M =", m, flush=True)
        oracle = _oracle_weight(container)[:, :cols].cuda()
        bias = (torch.randn(rows) * 0.01).to(torch.bfloat16).cuda() if rng.random() < 0.5 else None
        y = hip_lane.linear_mfma(buffers, shape=(rows, cols), x=x, bias=bias)
        torch.cuda.synchronize()
        hip_lane.check_errors(buffers)
        _check(y, x, oracle, bias, (rows, cols, bpp, tile_elements, m))
        done += 1


@pytest.mark.gpu
def test_linear_mfma_flags_a_corrupt_stream_and_refuses_other_tables():
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    torch.manual_seed(5)
    weight = (torch.randn(256, 512) * 0.02).to(torch.bfloat16)
    container = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager"))
    on_gpu = container.to("cuda")
    buffers = packed_buffers(on_gpu.buffers, LatticeBuffers)
    x = torch.randn(8, 512).to(torch.bfloat16).cuda()
    hip_lane.linear_mfma(buffers, shape=(256, 512), x=x, bias=None)
    torch.cuda.synchronize()
    hip_lane.check_errors(buffers)
    buffers.states.view(torch.int32)[0, 3] ^= 0x55                                     # a lane state the stream was not encoded from
    hip_lane.linear_mfma(buffers, shape=(256, 512), x=x, bias=None)
    with pytest.raises(ValueError):
        hip_lane.check_errors(buffers)
    # 8 bpp needs prob_bits 12 (rank/select tables): no two-level section, so the lane says it cannot take it.
    wide = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=8.0, execution_backend="eager")).to("cuda")
    wide_buffers = packed_buffers(wide.buffers, LatticeBuffers)
    assert not hip_lane.mfma_linear_usable(wide_buffers, (256, 512), x)
    with pytest.raises(ValueError):
        hip_lane.linear_mfma(wide_buffers, shape=(256, 512), x=x, bias=None)


@pytest.mark.gpu
def test_config_3_layer_in_fused_through_lds_mode_never_materialises_its_weight(monkeypatch):
    """Benchmark configuration 3 (W 3072 x 3072 @ 4 bpp + bias, X [M, 3072], seed 2) through the layer, M = 256, 1024 and the
    configuration's 4096: rel-L2 <= 1e-3 against F.linear on the oracle-decoded weight, with the decode-to-memory entry point
    made to raise for the duration (the mode's point is that the dense weight is never written)."""
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    torch.manual_seed(2)
    dense = torch.nn.Linear(3072, 3072, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(3072, 3072) * 0.02).to(torch.bfloat16))
    dense.bias.data.copy_((torch.randn(3072) * 0.01).to(torch.bfloat16))
    x = torch.randn(4096, 3072).to(torch.bfloat16).cuda()
    layer = ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager"),
                                            forward_mode="fused_through_lds").cuda()
    oracle = _oracle_weight(layer.weight.cpu()).cuda()
    bias = layer.bias.data

    def refuse(*args, **kwargs):
        raise AssertionError("fused_through_lds decoded the weight to memory")

    monkeypatch.setattr(hip_lane, "decode", refuse)
    for m in (256, 1024, 4096):
        print("case config 3 fused through LDS, M =", m, flush=True)
        part = x[:m].contiguous()
        before = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        y = layer(part)
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated()
        assert y.shape == (m, 3072) and y.dtype == torch.bfloat16
        _check(y, part, oracle, bias, ("config 3", m))
        if m == 256:
            # output + partial-sum planes + repacked activations: less than the 18.9 MB a dense copy of the weight would take
            assert peak - before < 3072 * 3072 * 2


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,tile_elements,activation_rows", [(768, 1024, None, (5, 100, 300)), (96, 288, 288, (33,)), (512, 3072, 4096, (64, 257))])
def test_int8_layer_in_fused_through_lds_mode_gives_the_bits_of_decode_then_gemm(rows, cols, tile_elements, activation_rows):
    """W8A8: the int8 codes are decoded inside the product (ep_hip_linear_fused_mfma_i8). Integer partial sums are exact and the
    epilogue is the int8 GEMM's, so the output must equal the decode_then_gemm layer's bit for bit, and both must equal the
    layer's definition f32(sum) * sa * sw + b (entropack/linear/quant_kernels.py:15-54 of the reference) rounded once."""
    from entropack_amd.linear import kernels
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    torch.manual_seed(rows)
    dense = torch.nn.Linear(cols, rows, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(rows, cols) * 0.02).to(torch.bfloat16))
    dense.bias.data.copy_((torch.randn(rows) * 0.01).to(torch.bfloat16))
    options = {} if tile_elements is None else {"tile_elements": tile_elements}
    config = ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager", **options)
    layers = {mode: ep.CompressedINT8Linear.from_linear(dense, config=config, forward_mode=mode).cuda() for mode in ("decode_then_gemm", "fused_through_lds")}
    layers["fused_through_lds"].load_state_dict(layers["decode_then_gemm"].state_dict())
    codes = layers["decode_then_gemm"].codes("cuda")
    for m in activation_rows:
        print("case int8 fused through LDS", (rows, cols, tile_elements), "M =", m, flush=True)
        x = torch.randn(m, cols).to(torch.bfloat16).cuda()
        expect = layers["decode_then_gemm"](x)
        got = layers["fused_through_lds"](x)
        torch.cuda.synchronize()
        assert got.shape == (m, rows) and got.dtype == torch.bfloat16
        assert torch.equal(got, expect), (m, (got.float() - expect.float()).abs().max().item())
        qa, sa = kernels.quantize_rows(x)
        exact = (qa.double() @ codes.double().T).float()
        definition = exact * sa.unsqueeze(1) * layers["decode_then_gemm"].weight_quant_scale.cuda().unsqueeze(0) + dense.bias.data.cuda().float()
        assert torch.equal(got, definition.to(torch.bfloat16))
    container = layers["fused_through_lds"]._container().to(device="cuda")
    hip_lane.check_errors(packed_buffers(container.buffers, LatticeBuffers))
