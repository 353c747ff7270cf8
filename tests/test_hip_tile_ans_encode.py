"""GPU parity of the lossless encoder on the device: `ep.compress(tensor_on_gpu, TileANSConfig(execution_backend="hip"))`
gives the container the CPU lane gives, byte for byte (all integer work: the byte histograms are exact and every
decision after them is the CPU lane's own code), for every dtype, ragged sizes, every option and every mix of raw and
coded byte lanes; and the result decodes to the input."""
import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.schemes.tile_ans import eager as tile_eager
from entropack_amd.schemes.tile_ans.format import TileBuffers

pytestmark = pytest.mark.gpu


def bits_of(tensor):
    tensor = tensor.detach().cpu().contiguous()
    if tensor.dtype == torch.bool:
        return tensor.numpy()
    return tensor.view(torch.uint8).numpy()


def same_container_on_both_lanes(tensor, **options):
    on_cpu = ep.compress(tensor, ep.TileANSConfig(execution_backend="eager", **options))
    on_gpu = ep.compress(tensor.cuda(), ep.TileANSConfig(execution_backend="hip", **options))
    assert on_cpu.compress_method == on_gpu.compress_method == "tile_ans"
    for key in TileBuffers._fields:
        mine, theirs = on_gpu.buffers[key], on_cpu.buffers[key]
        assert mine.device.type == "cuda" and mine.dtype == theirs.dtype and mine.shape == theirs.shape, key
        assert np.array_equal(bits_of(mine), bits_of(theirs)), key
    restored = ep.decompress(on_gpu, ep.TileANSConfig())
    assert restored.dtype == tensor.dtype and np.array_equal(bits_of(restored), bits_of(tensor))
    return on_gpu


def sample(dtype, shape, seed):
    generator = torch.Generator().manual_seed(seed)
    if dtype == torch.bool:
        return torch.rand(*shape, generator=generator) < 0.3
    if dtype.is_floating_point:
        return (torch.randn(*shape, generator=generator) * 0.05).to(dtype)
    if dtype == torch.uint8:
        return torch.randint(0, 40, shape, dtype=dtype, generator=generator)
    return (torch.randn(*shape, generator=generator) * 40).round().clamp(-120, 120).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int8, torch.uint8, torch.int16,
                                   torch.int32, torch.int64, torch.bool, torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("shape", [(1,), (31,), (33, 3), (257, 129), (3, 8192 + 17)])
def test_every_dtype_and_ragged_sizes(dtype, shape):
    print("case", dtype, shape, flush=True)
    same_container_on_both_lanes(sample(dtype, shape, len(shape) * 100 + shape[0]))


@pytest.mark.parametrize("options", [dict(tile_elements=400), dict(tile_elements=4096, probability_bits=12), dict(probability_bits=9),
                                     dict(raw_lane_threshold=0.0), dict(raw_lane_threshold=8.0, tile_elements=2048), dict(tile_elements=33)])
def test_across_options(options):
    print("case", options, flush=True)
    container = same_container_on_both_lanes(sample(torch.bfloat16, (300, 517), 77), **options)
    if options.get("raw_lane_threshold") == 0.0:
        assert container.buffers["lane_modes"].tolist() == [1, 1]
    steps = torch.randint(-300, 300, (123, 77), dtype=torch.int16, generator=torch.Generator().manual_seed(1)) * 16
    same_container_on_both_lanes(steps, **options)


@pytest.mark.parametrize("probability_bits", [0, 12])
def test_mixes_of_raw_and_coded_lanes(probability_bits):
    print("case", probability_bits, flush=True)
    generator = torch.Generator().manual_seed(21 + probability_bits)
    shape = (97, 1031)
    tensors = [
        torch.randint(-40000, 40000, shape, dtype=torch.int32, generator=generator),
        torch.randint(0, 200, shape, dtype=torch.int32, generator=generator),                   # three constant bytes (frequency 2^pb)
        (torch.randint(0, 256, shape, dtype=torch.int32, generator=generator) << 8) | torch.randint(0, 7, shape, dtype=torch.int32, generator=generator),
        torch.randint(0, 50000, shape, dtype=torch.int64, generator=generator),
        torch.randint(-128, 128, shape, dtype=torch.int8, generator=generator),
    ]
    seen = set()
    for tensor in tensors:
        for tile_elements in (256, 1000):
            container = same_container_on_both_lanes(tensor, tile_elements=tile_elements, probability_bits=probability_bits)
            modes = container.buffers["lane_modes"].tolist()
            seen.add((len(modes), modes.count(0)))
    counts = {coded for _, coded in seen}
    assert 0 in counts and counts & {2, 3, 4} and max(counts) > 4, seen


def test_a_view_that_does_not_start_on_16_bytes_and_the_refusals():
    whole = sample(torch.int8, (4099,), 5).cuda()
    view = whole[3:]
    assert view.data_ptr() % 16
    on_gpu = ep.compress(view, ep.TileANSConfig(execution_backend="hip"))
    on_cpu = ep.compress(view.cpu(), ep.TileANSConfig(execution_backend="eager"))
    for key in TileBuffers._fields:
        assert np.array_equal(bits_of(on_gpu.buffers[key]), bits_of(on_cpu.buffers[key])), key
    from entropack_amd.schemes.tile_ans import hip as tile_lane
    with pytest.raises(ValueError, match="on the GPU"):
        tile_lane.encode(weight=whole.cpu(), tile_elements=4096, probability_bits=0, raw_lane_threshold=7.9)
    with pytest.raises(ValueError, match="empty"):
        tile_lane.encode(weight=whole[:0], tile_elements=4096, probability_bits=0, raw_lane_threshold=7.9)


def test_full_size_weight_is_the_cpu_lanes_container():
    """8192 x 28672 bf16 (the lossless neighbour of the headline decode), default options."""
    generator = torch.Generator().manual_seed(4)
    weight = (torch.randn(8192, 28672, generator=generator) * 0.015).to(torch.bfloat16)
    same_container_on_both_lanes(weight)
