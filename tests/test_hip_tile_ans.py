"""GPU parity for the lossless `tile_ans` decode: the HIP lane against the reference-written fixtures and, on containers
this package's encoder wrote (byte-identical to the reference's on the fixtures), against the input itself and the
CPU oracle, from one element to 8192 x 28672."""
import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.schemes.base import packed_buffers
from entropack_amd.schemes.tile_ans import hip as tile_lane
from entropack_amd.schemes.tile_ans.format import TileBuffers
from oracle import c_oracle
from test_tile_ans_golden import TileGolden, tile_names

pytestmark = pytest.mark.gpu

_BITS = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def bits_of(tensor):
    tensor = tensor.detach().contiguous()
    if tensor.dtype == torch.bool:
        return tensor.to(torch.uint8).cpu().numpy()
    return tensor.view(_BITS[tensor.element_size()]).cpu().numpy()


@pytest.mark.parametrize("name", tile_names())
def test_decompress_matches_reference_bits(name):
    print("case", name, flush=True)
    golden = TileGolden(name)
    container = ep.CompressedTensor.unpack(torch.from_numpy(golden.quant_state.copy()).cuda())
    restored = ep.decompress(container, ep.TileANSConfig(execution_backend="hip"))
    torch.cuda.synchronize()
    tile_lane.check_errors(packed_buffers(container.buffers, TileBuffers))
    assert restored.shape == golden.shape and restored.dtype == golden.dtype and restored.device.type == "cuda"
    want = golden.weight_bits if golden.dtype != torch.bool else golden.weight_bits.astype(np.uint8)
    assert np.array_equal(bits_of(restored), want.reshape(golden.shape))


def round_trip(tensor, **options):
    container = ep.compress(tensor, ep.TileANSConfig(execution_backend="eager", **options))
    assert container.compress_method == "tile_ans"
    on_gpu = container.to("cuda")
    restored = ep.decompress(on_gpu, ep.TileANSConfig())            # "auto" resolves to hip on this box
    torch.cuda.synchronize()
    tile_lane.check_errors(packed_buffers(on_gpu.buffers, TileBuffers))
    assert restored.shape == tensor.shape and restored.dtype == tensor.dtype
    assert np.array_equal(bits_of(restored), bits_of(tensor))
    return container


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int8, torch.uint8, torch.int16, torch.int32,
                                   torch.int64, torch.bool, torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("shape", [(1,), (31,), (33, 3), (257, 129), (5, 4096), (3, 8192 + 17)])
def test_round_trip_every_dtype_and_ragged_sizes(dtype, shape):
    print("case", dtype, shape, flush=True)
    torch.manual_seed(hash((str(dtype), shape)) % 1000)
    if dtype == torch.bool:
        tensor = torch.rand(*shape) < 0.3
    elif dtype.is_floating_point:
        tensor = (torch.randn(*shape) * 0.05).to(dtype)
    else:
        tensor = (torch.randn(*shape) * 40).round().clamp(-120, 120).to(dtype) if dtype != torch.uint8 else torch.randint(0, 40, shape, dtype=dtype)
    round_trip(tensor)


@pytest.mark.parametrize("options", [dict(tile_elements=400), dict(tile_elements=4096, probability_bits=12), dict(probability_bits=9),
                                     dict(raw_lane_threshold=0.0), dict(raw_lane_threshold=8.0, tile_elements=2048)])
def test_round_trip_across_options(options):
    print("case", options, flush=True)
    torch.manual_seed(77)
    container = round_trip((torch.randn(300, 517) * 0.02).to(torch.bfloat16), **options)
    if options.get("raw_lane_threshold") == 0.0:
        assert container.buffers["lane_modes"].tolist() == [1, 1]          # nothing coded: a plain unpacking of the words
    steps = torch.randint(-300, 300, (123, 77), dtype=torch.int16) * 16        # both byte lanes coded
    container = round_trip(steps, **options)
    if options.get("raw_lane_threshold", 7.9) > 0.0:
        assert container.buffers["lane_modes"].tolist() == [0, 0]


def test_model_weight_sizes_match_the_oracle_and_the_input():
    """A 4096 x 4096 bf16 weight (8192-element tiles, raw low byte + coded high byte) and a float32 one, against the oracle."""
    for dtype, shape in ((torch.bfloat16, (4096, 4096)), (torch.float32, (1024, 3072)), (torch.int8, (2048, 4096))):
        print("case", dtype, shape, flush=True)
        torch.manual_seed(5)
        tensor = (torch.randn(*shape) * 0.02).to(dtype) if dtype.is_floating_point else (torch.randn(*shape) * 30).round().clamp(-127, 127).to(dtype)
        container = round_trip(tensor)
        host = {}
        for key, value in container.buffers.items():
            if value.dtype in (torch.uint16, torch.uint32):
                signed = value.view(torch.int16 if value.dtype == torch.uint16 else torch.int32).numpy()
                host[key] = signed.view(np.uint16 if value.dtype == torch.uint16 else np.uint32)
            else:
                host[key] = value.numpy()
        expect = c_oracle.tile_ans_decode(host, tensor.element_size(), threads=8)
        assert np.array_equal(expect, tensor.contiguous().view(torch.uint8).numpy().reshape(-1))
        ratio = container.storage_nbytes() / (tensor.numel() * tensor.element_size())
        assert ratio < 0.9                                                    # gaussian weights do compress (float32: 0.84)


def test_full_size_8192x28672_bf16_is_lossless():
    torch.manual_seed(4)
    tensor = (torch.randn(8192, 28672) * 0.015).to(torch.bfloat16)
    container = round_trip(tensor)
    assert container.buffers["lane_modes"].tolist() == [1, 0] and int(container.buffers["layout"][0]) == 8192


def test_corrupt_stream_sets_the_error_flag_and_stays_in_bounds():
    golden = TileGolden("int8_128x100_auto")
    container = ep.CompressedTensor.unpack(torch.from_numpy(golden.quant_state.copy()).cuda())
    buffers = dict(container.buffers)
    states = buffers["states"].clone()
    states.view(torch.int32)[0, 3] += 12345                                   # a wrong initial state derails that lane
    buffers["states"] = states
    lattice = TileBuffers(**buffers)
    tile_lane.decode(lattice, dtype=torch.int8)
    with pytest.raises(ValueError, match="decode error"):
        tile_lane.check_errors(lattice)
    tile_lane.check_errors(lattice)                                           # the flag was cleared by the read


def test_one_symbol_lane_at_twelve_bits():
    """A coded lane whose table holds a single symbol has frequency 4096, which the LDS entries of the one-coded-lane
    kernel cannot hold; those workgroups decode stream by stream. Low byte random (raw), high byte constant (coded)."""
    torch.manual_seed(11)
    values = torch.randint(0, 256, (37, 1000), dtype=torch.int16) + 0x2A00
    container = round_trip(values, probability_bits=12, tile_elements=4096)
    assert container.buffers["lane_modes"].tolist() == [1, 0]
    table = container.buffers["decode_tables"].view(torch.int32)[1]
    assert int(((table >> 8) & 0xFFF).max()) == 0                       # 4096 is stored as 0
    constant = torch.full((9000,), 7, dtype=torch.int8)
    round_trip(constant, probability_bits=12, tile_elements=2048)


@pytest.mark.parametrize("tile_elements", [256, 320, 1000, 4096])
def test_one_coded_lane_tile_sizes(tile_elements):
    """Whole 256-element chunks take the wide-store path, other tile sizes and the last short tile the group path."""
    print("case", tile_elements, flush=True)
    torch.manual_seed(tile_elements)
    for dtype in (torch.bfloat16, torch.float32, torch.int8, torch.int64):
        if dtype == torch.int64:       # seven random bytes under a peaked top byte: 7 raw lanes + 1 coded
            tensor = torch.randint(0, 1 << 56, (70, 999), dtype=dtype) + ((torch.randn(70, 999) * 6).round().to(dtype).clamp(-100, 100) << 56)
        else:
            tensor = (torch.randn(70, 999) * 0.03).to(dtype) if dtype.is_floating_point else (torch.randn(70, 999) * 20).round().to(dtype)
        container = round_trip(tensor, tile_elements=tile_elements)
        assert sum(1 for mode in container.buffers["lane_modes"].tolist() if mode == 0) <= 1     # 0 where the states cost too much


def test_output_address_need_not_be_aligned():
    """Through the C ABI with an output 2 bytes off a 16-byte boundary: the same bytes."""
    torch.manual_seed(3)
    tensor = (torch.randn(64, 4096) * 0.02).to(torch.bfloat16)
    container = ep.compress(tensor, ep.TileANSConfig(execution_backend="eager")).to("cuda")
    buffers = packed_buffers(container.buffers, TileBuffers)
    from entropack_amd.backends import hip as backend
    modes = np.asarray(buffers.lane_modes.cpu().tolist(), dtype=np.uint8)
    tile_elements, prob_bits, lanes, elements = (int(v) for v in buffers.layout.tolist())
    room = torch.zeros(elements * lanes + 64, dtype=torch.uint8, device="cuda")
    error = torch.zeros(1, dtype=torch.int32, device="cuda")
    for shift in (0, 2, 6):
        room.zero_()
        backend.check("ep_hip_decode_tile_ans", backend.library().ep_hip_decode_tile_ans(
            backend.pointer(buffers.payload), buffers.payload.numel(), buffers.offsets.data_ptr(), backend.pointer(buffers.states),
            buffers.decode_tables.data_ptr(), modes.ctypes.data, tile_elements, prob_bits, lanes, elements,
            room.data_ptr() + shift, error.data_ptr(), backend.current_stream(room.device)))
        torch.cuda.synchronize()
        assert int(error.item()) == 0
        got = room[shift:shift + elements * lanes].cpu().numpy()
        assert np.array_equal(got, tensor.contiguous().view(torch.uint8).numpy().reshape(-1))
        assert int(room[shift + elements * lanes:].max()) == 0 and int(room[:shift].sum()) == 0


@pytest.mark.parametrize("mode", ["decode_then_gemm", "fused"])
def test_compressed_linear_with_lossless_weights(mode):
    """`CompressedLinear.from_linear(linear)` with no config stores the weight with tile_ans (the reference's default
    for bfloat16): the layer's dense weight is the original one bit for bit, and its forward is the dense forward."""
    torch.manual_seed(8)
    dense = torch.nn.Linear(1024, 768, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(768, 1024) * 0.02).to(torch.bfloat16))
    layer = ep.CompressedLinear.from_linear(dense, forward_mode=mode)
    assert layer.weight.compress_method == "tile_ans" and layer.compressed_bits < 12.0
    state = layer.state_dict()
    fresh = ep.CompressedLinear(1024, 768, forward_mode=mode)
    fresh.load_state_dict(state)
    fresh = fresh.cuda()
    assert torch.equal(fresh.dequantize("cuda").cpu().view(torch.int16), dense.weight.data.view(torch.int16))
    for rows in (1, 7, 300):
        x = torch.randn(rows, 1024).to(torch.bfloat16).cuda()
        expect = torch.nn.functional.linear(x.float(), dense.weight.data.cuda().float(), dense.bias.data.cuda().float())
        got = fresh(x)
        error = ((got.float() - expect).norm() / expect.norm()).item()
        assert got.dtype == torch.bfloat16 and error <= 4e-3, (rows, error)            # one bf16 rounding of the output


@pytest.mark.parametrize("probability_bits", [0, 9, 12])
def test_several_coded_lanes_and_none(probability_bits):
    """Containers with two, three and four coded lanes (the tile kernel carries one rANS state per coded lane and half),
    with none (every lane raw: a byte-plane interleave), and with more than four (general kernel); whole 256-element
    chunks, other tile sizes and short last tiles. At 12 bits a constant lane has frequency 4096 (stream-by-stream path)."""
    print("case", probability_bits, flush=True)
    torch.manual_seed(21 + probability_bits)
    shape = (97, 1031)
    small16 = torch.randint(-300, 300, shape, dtype=torch.int16)                       # both bytes structured
    small32 = torch.randint(-40000, 40000, shape, dtype=torch.int32)                   # two structured bytes + two near-constant
    tiny32 = torch.randint(0, 200, shape, dtype=torch.int32)                           # one structured + three constant
    mixed32 = (torch.randint(0, 256, shape, dtype=torch.int32) << 8) | torch.randint(0, 7, shape, dtype=torch.int32)   # raw in the middle
    ids64 = torch.randint(0, 50000, shape, dtype=torch.int64)                          # six constant bytes: more than four coded lanes
    noise = torch.randint(-128, 128, shape, dtype=torch.int8)
    seen = set()
    for tensor in (small16, small32, tiny32, mixed32, ids64, noise):
        for tile_elements in (256, 1000, 4096):
            container = round_trip(tensor, tile_elements=tile_elements, probability_bits=probability_bits)
            modes = container.buffers["lane_modes"].tolist()
            seen.add((len(modes), modes.count(0)))
    counts = {coded for _, coded in seen}
    assert 0 in counts and counts & {2, 3, 4} and max(counts) > 4, seen          # all raw, the multi-lane tile kernel, the general kernel
