"""GPU parity of the device encoder (`ep_hip_encode_*` through the hip lane) against the CPU encoder, which is itself
bit-identical to the reference's on the golden containers (test_encoder_golden.py).

Stage by stage, from the same row RMS and lattice scale: coset bits, fields, stream statistics, histograms, states,
offsets and payload must be equal bit for bit. The refitted row scales are float32 sums added in another order than
torch's on the CPU: equal to 1e-5 relative (stated where it is checked), and equal bit for bit on inputs whose sums are
exact in float32, on which the whole container must come out byte-identical from both lanes."""
import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.schemes.lattice_rans import eager, hip_encode
from entropack_amd.schemes.lattice_rans import hip as hip_lane
from entropack_amd.schemes.lattice_rans.format import LatticeBuffers, validate_packed
from oracle import c_oracle

pytestmark = pytest.mark.gpu


def matrix(seed, rows, cols, sigma=0.02, outliers=False):
    generator = torch.Generator().manual_seed(seed)
    weight = torch.randn(rows, cols, generator=generator) * sigma
    if outliers:
        index = torch.randperm(rows * cols, generator=generator)[: max(1, rows * cols // 1000)]
        weight.view(-1)[index] *= 20.0
    return weight.contiguous()


def both_quantizers(x_cpu, rms_cpu=None):
    rms_cpu = eager.row_rms(x_cpu, x_cpu.dtype) if rms_cpu is None else rms_cpu
    return eager.HostQuantizer(x_cpu, rms_cpu), hip_encode.DeviceQuantizer(x_cpu.cuda(), rms_cpu.cuda())


def assert_same_quantisation(q_host, q_device):
    assert np.array_equal(q_device.coset.cpu().numpy(), q_host.coset)
    assert np.array_equal(q_device.fields.cpu().numpy(), q_host.fields)
    stats = q_host.stats()
    assert np.array_equal(q_device.stats(), stats)
    for mine, theirs in zip(q_device.histograms(stats), q_host.histograms(stats)):
        assert np.array_equal(mine, theirs)


@pytest.mark.parametrize("rows,cols,scale,sigma,outliers", [
    (1, 8, 0.5, 0.02, False),
    (3, 40, 0.31, 0.02, False),
    (64, 512, 0.12, 0.02, False),
    (257, 1032, 0.7, 1.0, False),
    (128, 4096, 0.05, 0.02, True),
    (1024, 3072, 0.2, 0.02, False),
])
def test_quantise_matches_the_cpu_encoder(rows, cols, scale, sigma, outliers):
    host, device = both_quantizers(matrix(rows * 7 + cols, rows, cols, sigma, outliers))
    assert_same_quantisation(host.quantize(scale), device.quantize(scale))


def test_quantise_of_a_row_subsample():
    host, device = both_quantizers(matrix(5, 300, 256))
    picked = np.ascontiguousarray(torch.randperm(300, generator=torch.Generator().manual_seed(9))[:77].numpy(), dtype=np.int64)
    assert_same_quantisation(host.quantize(0.25, picked), device.quantize(0.25, picked))
    with pytest.raises(IndexError):
        device.quantize(0.25, np.array([0, 300], dtype=np.int64))


def test_quantise_breaks_ties_like_the_cpu_encoder():
    """Coordinates on quarter steps with a row 'RMS' of 1 and a scale of 1/2: every division is exact, so roundings to
    even, the choice of the coordinate to move and ties between the two cosets all occur, thousands of times."""
    generator = torch.Generator().manual_seed(11)
    y = torch.randint(-14, 15, (96, 1024), generator=generator).float() * 0.25
    y[:, :64] = torch.randint(-3, 4, (96, 64), generator=generator).float() * 0.5      # half steps only: many exact coset ties
    x = (y * 0.5).contiguous()
    host, device = both_quantizers(x, torch.ones(96, 1))
    q_host, q_device = host.quantize(0.5), device.quantize(0.5)
    assert 0 < int(q_host.coset.sum()) < q_host.coset.size
    assert_same_quantisation(q_host, q_device)


def test_quantise_of_zeros_and_of_one_coset_only():
    host, device = both_quantizers(torch.zeros(4, 64), torch.full((4, 1), 1e-12))
    q_host, q_device = host.quantize(1.0), device.quantize(1.0)
    assert_same_quantisation(q_host, q_device)
    assert q_device.stats()[0].tolist() == [32, 0, 0] and int(q_device.stats()[2, 0]) == 0      # no vector of coset 1
    assert np.array_equal(device.refit(q_device, 1.0).cpu().numpy(), host.refit(q_host, 1.0).numpy())
    halves = torch.full((2, 16), 0.5)
    host, device = both_quantizers(halves, torch.ones(2, 1))
    q_host, q_device = host.quantize(1.0), device.quantize(1.0)
    assert int(q_host.coset.min()) == 1
    assert_same_quantisation(q_host, q_device)


@pytest.mark.parametrize("rows,cols,scale,prob_bits,tile_elements", [
    (1, 8, 0.5, 11, 16384),           # one vector
    (8, 256, 0.3, 9, 288),            # tiles of 32 vectors, all whole
    (9, 264, 0.3, 10, 300),           # tiles of 33 vectors, ragged last tile
    (64, 1000, 0.12, 11, 16384),      # one ragged tile
    (300, 1024, 0.1, 12, 16384),
    (512, 2048, 0.02, 14, 8208),      # wide alphabets
    (256, 4096, 0.05, 15, 4104),
    (2048, 3072, 0.2, 11, 16384),
])
def test_stream_encode_matches_the_cpu_encoder(rows, cols, scale, prob_bits, tile_elements):
    host, device = both_quantizers(matrix(rows + cols + prob_bits, rows, cols, outliers=prob_bits >= 14))
    q_host, q_device = host.quantize(scale), device.quantize(scale)
    payload, states, offsets, meta, freq = eager.encode_streams(q_host, prob_bits, tile_elements)
    got_payload, got_states, got_offsets, got_meta, got_freq = hip_encode.encode_streams(q_device, prob_bits, tile_elements)
    assert np.array_equal(got_meta, meta) and np.array_equal(got_freq, freq)
    assert np.array_equal(got_offsets.view(torch.int32).cpu().numpy().view(np.uint32), offsets)
    assert np.array_equal(got_states.view(torch.int32).cpu().numpy().view(np.uint32), states)
    assert np.array_equal(got_payload.view(torch.int16).cpu().numpy().view(np.uint16), payload)


def test_refitted_row_scales():
    """float32 sums in another order than torch's: 1e-5 relative against the CPU lane, and against the float64 value of
    the same definition."""
    x = matrix(21, 192, 4096)
    host, device = both_quantizers(x)
    q_host, q_device = host.quantize(0.15), device.quantize(0.15)
    got = device.refit(q_device, 0.15).cpu()
    assert torch.allclose(got, host.refit(q_host, 0.15), rtol=1e-5, atol=0.0)
    levels = q_host.levels().reshape(192, 4096).double()
    exact = (x.double() * levels).sum(1) / levels.square().sum(1)
    assert torch.allclose(got.double(), exact, rtol=1e-5, atol=0.0)


def host_arrays(buffers):
    out = {}
    for key, value in zip(LatticeBuffers._fields, buffers):
        value = value.detach().cpu()
        if value.dtype == torch.uint16:
            out[key] = value.view(torch.int16).numpy().view(np.uint16)
        elif value.dtype == torch.uint32:
            out[key] = value.view(torch.int32).numpy().view(np.uint32)
        else:
            out[key] = value.numpy()
    return out


def test_exactly_summable_weights_give_the_cpu_lanes_container():
    """Entries on multiples of 1/64 within +-2 and 256 columns: every float32 row sum either lane forms is exact in any
    order, so from the CPU lane's row RMS (its square root is torch's vectorised one, which no other routine
    reproduces) the scale search, the refitted scales and with them the whole container must be byte-identical."""
    generator = torch.Generator().manual_seed(3)
    weight = (torch.randn(192, 256, generator=generator) * 0.6).clamp(-2, 2).mul(64).round().div(64).contiguous()
    on_cpu = host_arrays(eager.encode(weight=weight, target_bpp=4.0, prob_bits=None, tile_elements=4104))
    rms = eager.row_rms(weight, weight.dtype)
    on_gpu = host_arrays(hip_encode.encode_normalised(weight.cuda(), rms.cuda(), target_bpp=4.0, prob_bits=None, tile_elements=4104))
    for key in LatticeBuffers._fields:
        assert np.array_equal(on_gpu[key], on_cpu[key]), key
    assert torch.equal(hip_encode.row_rms(weight.cuda(), weight.dtype).cpu(), weight.square().mean(1, keepdim=True).double().sqrt().float())


def test_random_weights_with_the_cpu_lanes_row_rms():
    """The same on an ordinary weight: everything but the refitted scales is byte-identical, the scales to 1e-5."""
    weight = matrix(17, 512, 1024)
    on_cpu = host_arrays(eager.encode(weight=weight, target_bpp=3.0, prob_bits=None, tile_elements=16384))
    rms = eager.row_rms(weight, weight.dtype)
    on_gpu = host_arrays(hip_encode.encode_normalised(weight.cuda(), rms.cuda(), target_bpp=3.0, prob_bits=None, tile_elements=16384))
    for key in LatticeBuffers._fields:
        if key != "scales":
            assert np.array_equal(on_gpu[key], on_cpu[key]), key
    assert np.allclose(on_gpu["scales"], on_cpu["scales"], rtol=1e-5, atol=0.0)


@pytest.mark.parametrize("rows,cols,bpp,dtype", [
    (256, 256, 3.5, torch.bfloat16),
    (1024, 1024, 4.0, torch.bfloat16),
    (300, 200, 5.0, torch.float32),
    (512, 4096, 2.3, torch.float16),
    (2048, 3072, 8.0, torch.bfloat16),
])
def test_compress_on_the_device_end_to_end(rows, cols, bpp, dtype):
    """`ep.compress` of a tensor on the GPU: a valid container at the asked rate, decoded by the hip lane bit for bit as
    the CPU oracle decodes it, and as close to the weight as the CPU lane's container is."""
    weight = matrix(rows + cols, rows, cols).to(dtype)
    config = ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="hip")
    container = ep.compress(weight.cuda(), config)
    assert all(value.device.type == "cuda" for value in container.buffers.values())
    buffers = LatticeBuffers(**{key: container.buffers[key] for key in LatticeBuffers._fields})
    validate_packed(dict(container.buffers), (rows, cols), dtype)
    reference = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager"))
    assert abs(container.actual_bpp - reference.actual_bpp) <= 0.01 * reference.actual_bpp

    restored = ep.decompress(container, config)
    torch.cuda.synchronize()
    padded = int(container.buffers["layout"][0])
    name = str(dtype).removeprefix("torch.")
    expect = c_oracle.decode(host_arrays(buffers), (rows, padded), name, threads=8)[:, :cols]
    if dtype in (torch.bfloat16, torch.float16):             # the oracle returns 16-bit floats as their bit patterns
        got = restored.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    else:
        got = restored.cpu().numpy()
    assert np.array_equal(got, expect)

    def relative_error(tensor):
        return float((tensor.float().cpu() - weight.float()).norm() / weight.float().norm())

    theirs = relative_error(ep.decompress(reference.to("cuda"), config))
    assert abs(relative_error(restored) - theirs) <= 0.01 * theirs


def test_hip_lane_takes_a_cpu_tensor_to_the_device_and_back():
    weight = matrix(2, 64, 128).to(torch.bfloat16)
    container = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="hip"))
    assert all(value.device.type == "cpu" for value in container.buffers.values())
    with pytest.raises(ValueError, match="on the GPU"):
        hip_encode.encode(weight=weight.float(), target_bpp=4.0, prob_bits=None, tile_elements=16384)
    with pytest.raises(ValueError, match="multiple of 8"):
        hip_encode.encode(weight=torch.zeros(4, 12, device="cuda"), target_bpp=4.0, prob_bits=None, tile_elements=16384)


def test_row_refinement_on_the_device():
    """`row_rdo_iterations` on the device lane: the same pass over the device's kernels. Its float32 row sums (prices,
    squared errors) are added in another order than the CPU lane's, so a row on the fence may choose differently: the
    container is valid, decodes as the oracle decodes it, and has the CPU lane's rate and error to 1 %; and it beats
    the plain encode's error at no more bytes, which is what the pass is for."""
    weight = (matrix(33, 128, 256) * torch.logspace(-1, 1, 128).unsqueeze(1)).to(torch.bfloat16)
    options = dict(target_bpp=3.0, prob_bits=None, tile_elements=16384)
    x = weight.float().contiguous()
    rms = eager.row_rms(x, weight.dtype)
    host, device = both_quantizers(x, rms)
    q_host, q_device = host.quantize(0.3), device.quantize(0.3)
    scales_host, sse_host = host.refit_with_error(q_host, 0.3)
    scales_device, sse_device = device.refit_with_error(q_device, 0.3)
    assert torch.allclose(scales_device.cpu(), scales_host, rtol=1e-5, atol=0.0)
    assert torch.allclose(sse_device.cpu(), sse_host, rtol=1e-3, atol=0.0)        # a difference of two nearly equal sums

    def error_of(buffers):
        dense = hip_lane.decode(buffers, shape=(128, 256), dtype=torch.bfloat16)
        torch.cuda.synchronize()
        hip_lane.check_errors(buffers)
        expect = c_oracle.decode(host_arrays(buffers), (128, 256), "bfloat16", threads=4)
        assert np.array_equal(dense.view(torch.int16).cpu().numpy().view(np.uint16), expect)
        return float((dense.float().cpu() - x).square().sum())

    def size_of(buffers):
        return sum(t.numel() * t.element_size() for t in buffers)

    plain = hip_encode.encode_normalised(x.cuda(), rms.cuda(), **options)
    refined = hip_encode.encode_normalised(x.cuda(), rms.cuda(), row_rdo_iterations=2, **options)
    on_cpu = LatticeBuffers(*(t.cuda() for t in eager.encode(weight=weight, row_rdo_iterations=2, **options)))
    validate_packed(dict(zip(LatticeBuffers._fields, refined)), (128, 256), torch.bfloat16)
    assert error_of(refined) < error_of(plain) and size_of(refined) <= size_of(plain) + 16
    assert abs(size_of(refined) - size_of(on_cpu)) <= 0.01 * size_of(on_cpu)
    assert abs(error_of(refined) - error_of(on_cpu)) <= 0.01 * error_of(on_cpu)


def test_layers_compress_device_weights_on_the_device(monkeypatch):
    """`CompressedLinear.from_linear` of a layer on the GPU never visits the CPU lane, and its forward is the dense
    product with the weight the container decodes to."""
    def refuse(**kwargs):
        raise AssertionError("the CPU lane was asked to encode a device tensor")
    monkeypatch.setattr(eager, "encode", refuse)
    torch.manual_seed(5)
    dense = torch.nn.Linear(512, 256, dtype=torch.bfloat16, device="cuda")
    layer = ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0))
    assert layer.weight.buffers["payload"].device.type == "cuda"
    x = torch.randn(32, 512, dtype=torch.bfloat16, device="cuda")
    restored = ep.decompress(layer.weight, ep.EntroPackLossyConfig(execution_backend="hip"))
    assert torch.equal(layer(x), torch.nn.functional.linear(x, restored, dense.bias))
    original = dense.weight.detach().float()
    relative = float((restored.float() - original).norm() / original.norm())
    assert relative < 0.1
    codes_layer = ep.CompressedINT8Linear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0))
    assert codes_layer.weight.buffers["payload"].device.type == "cuda"
