"""GPU parity, part 1: the HIP lane against the dense tensors the reference's decoder wrote (tests/golden)."""
import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.backends import hip as hip_backend
from entropack_amd.schemes.lattice_rans import hip as hip_lane
from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
from conftest import Golden, golden_names
from oracle import c_oracle

pytestmark = pytest.mark.gpu

_VIEW = {"bfloat16": torch.int16, "float16": torch.int16, "float32": torch.int32, "int8": torch.uint8}
KINDS = [hip_backend.TABLE_GLOBAL64, hip_backend.TABLE_LDS_BYTE, hip_backend.TABLE_LDS_WIDE, hip_backend.TABLE_LDS_RANK,
         hip_backend.TABLE_LDS_SYM]


def _container(golden, device="cuda"):
    return ep.CompressedTensor.unpack(torch.from_numpy(golden.quant_state.copy()).to(device))


@pytest.fixture(autouse=True)
def _reset_force():
    yield
    hip_lane.FORCE_TABLE_KIND = None


@pytest.mark.parametrize("kind", KINDS, ids=["global64", "lds_byte", "lds_wide", "lds_rank", "lds_sym"])
@pytest.mark.parametrize("name", golden_names())
def test_decompress_matches_reference_bits(name, kind):
    print(f"case {name} kind {kind}", flush=True)
    golden = Golden(name)
    hip_lane.FORCE_TABLE_KIND = kind
    compressed = _container(golden)
    try:
        restored = ep.decompress(compressed, ep.EntroPackLossyConfig(execution_backend="hip"))
    except hip_backend.HipError as error:
        if error.status == hip_backend.EUNSUPPORTED:
            pytest.skip("container does not qualify for this table kind")
        raise
    torch.cuda.synchronize()
    buffers = LatticeBuffers(**{k: compressed.buffers[k] for k in LatticeBuffers._fields})
    hip_lane.check_errors(buffers)
    assert hip_lane.plan_of(buffers).desc.table_kind == kind
    assert restored.shape == golden.shape and str(restored.dtype) == "torch." + golden.dtype
    got = restored.contiguous().view(_VIEW[golden.dtype]).cpu().numpy()
    assert np.array_equal(got, golden.restored_bits)


@pytest.mark.parametrize("name", ["outlier_128x256_bf16_4p0", "hi_96x512_bf16_8p0", "pb9_64x128_bf16_1p5"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.int8, torch.uint8, torch.int16,
                                   torch.int32, torch.int64, torch.bool, torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("kind", [None, hip_backend.TABLE_LDS_RANK, hip_backend.TABLE_LDS_SYM], ids=["auto", "lds_rank", "lds_sym"])
def test_every_store_kind_matches_oracle(name, dtype, kind):
    print(f"case {name} dtype {dtype} kind {kind}", flush=True)
    golden = Golden(name)
    hip_lane.FORCE_TABLE_KIND = kind
    compressed = _container(golden)
    buffers = {k: v for k, v in compressed.buffers.items()}
    if dtype in (torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64, torch.bool):
        buffers["scales"] = buffers["scales"] * 900.0          # spread the values over and beyond the int8 range
    try:
        dense = hip_lane.decode(LatticeBuffers(**buffers), shape=golden.shape, dtype=dtype)
    except hip_backend.HipError as error:
        if kind is not None and error.status == hip_backend.EUNSUPPORTED:
            pytest.skip("container does not qualify for this table kind")
        raise
    torch.cuda.synchronize()
    host = {k: v.cpu().numpy() if v.dtype not in (torch.uint16, torch.uint32) else
            v.cpu().view(torch.int16 if v.dtype == torch.uint16 else torch.int32).numpy().view(np.uint16 if v.dtype == torch.uint16 else np.uint32)
            for k, v in buffers.items()}
    if dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        reference = torch.from_numpy(c_oracle.decode(host, golden.shape, "float32"))
        limit = float(torch.finfo(dtype).max)
        expect = reference.clamp(-limit, limit).to(dtype).view(torch.uint8).numpy()
        assert np.array_equal(dense.view(torch.uint8).cpu().numpy(), expect)
        return
    name_of = str(dtype).removeprefix("torch.")
    expect = c_oracle.decode(host, golden.shape, name_of)
    got = dense.cpu()
    if dtype in (torch.bfloat16, torch.float16):
        got = got.view(torch.int16).numpy().view(np.uint16)
    elif dtype == torch.bool:
        got = got.numpy().astype(np.uint8)
    elif dtype == torch.float32:
        got, expect = got.view(torch.int32).numpy(), expect.view(np.int32)
    else:
        got = got.numpy()
    assert np.array_equal(got, expect)


def test_corrupt_payload_sets_the_error_flag_and_stays_in_bounds():
    golden = Golden("ragged_66x200_bf16_4p0")
    for kind in (hip_backend.TABLE_GLOBAL64, hip_backend.TABLE_LDS_BYTE, hip_backend.TABLE_LDS_RANK, hip_backend.TABLE_LDS_SYM):
        hip_lane.FORCE_TABLE_KIND = kind
        compressed = _container(golden)
        buffers = dict(compressed.buffers)
        states = buffers["states"].clone()
        states.view(torch.int32)[0, 3] += 12345              # a wrong initial state derails that lane
        buffers["states"] = states
        lattice = LatticeBuffers(**buffers)
        hip_lane.decode(lattice, shape=golden.shape, dtype=torch.bfloat16)
        with pytest.raises(ValueError, match="decode error"):
            hip_lane.check_errors(lattice)
        hip_lane.check_errors(lattice)                         # the flag was cleared by the read


@pytest.mark.parametrize("damage", ["payload", "boundaries", "order"])
def test_damaged_streams_decode_to_completion_with_the_flag_set(damage):
    """Streams that are readable but wrong (flipped payload words, tile boundaries moved inside the payload, two
    tiles' boundaries swapped) take every kernel through its window refills with positions the encoder never made:
    the decode must finish, and such damage is reported."""
    golden = Golden("c1_256x256_bf16_3p5")
    generator = torch.Generator().manual_seed(5)
    for kind in (hip_backend.TABLE_GLOBAL64, hip_backend.TABLE_LDS_BYTE, hip_backend.TABLE_LDS_RANK, hip_backend.TABLE_LDS_SYM):
        hip_lane.FORCE_TABLE_KIND = kind
        try:
            compressed = _container(golden)
            buffers = dict(compressed.buffers)
            if damage == "payload":
                payload = buffers["payload"].clone().view(torch.int16)
                where = torch.randint(0, payload.numel(), (max(1, payload.numel() // 50),), generator=generator)
                payload[where.to(payload.device)] ^= 0x5A5A
                buffers["payload"] = payload.view(torch.uint16)
            else:
                offsets = buffers["offsets"].clone().view(torch.int32)
                assert offsets.numel() > 4
                if damage == "boundaries":
                    offsets[1:-1] += 7                              # every inner boundary 7 words too high, still ordered
                    offsets[1:-1] = torch.minimum(offsets[1:-1], offsets[-1])
                else:
                    offsets[[1, 2]] = offsets[[2, 1]]                   # tile 1 now ends before it begins
                buffers["offsets"] = offsets.view(torch.uint32)
            lattice = LatticeBuffers(**buffers)
            out = hip_lane.decode(lattice, shape=golden.shape, dtype=torch.bfloat16)
            torch.cuda.synchronize()
            assert tuple(out.shape)[0] == golden.shape[0]
            with pytest.raises(ValueError, match="decode error"):
                hip_lane.check_errors(lattice)
        finally:
            hip_lane.FORCE_TABLE_KIND = None

