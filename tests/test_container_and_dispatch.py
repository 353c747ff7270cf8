"""Host logic that needs no GPU: container blob layout, configs, registry dispatch, the C-ABI surface, plan choice."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd import registry
from entropack_amd.backends import hip as hip_backend
from entropack_amd.compression.compressed_tensor import pack_quant_state, parse_quant_state
from entropack_amd.schemes.config import validate_config
from entropack_amd.schemes.lattice_rans import format as fmt
from conftest import ROOT, Golden


def _blob(golden):
    return torch.from_numpy(golden.quant_state.copy())


def test_blob_parses_to_the_reference_buffers(golden):
    container = ep.CompressedTensor.unpack(_blob(golden))
    assert tuple(container.shape) == golden.shape
    assert str(container.encoded_dtype) == "torch." + golden.dtype
    assert container.compress_method == "lattice_rans" and not container.lossless
    assert container.actual_bpp == pytest.approx(golden.actual_bpp, abs=0)
    assert list(container.buffers) == list(fmt.PACKED_KEYS)
    for key, expect in golden.buffers.items():
        got = container.buffers[key]
        assert got.dtype == fmt.BUFFER_DTYPES[key]
        assert got.data_ptr() % 16 == 0 or got.numel() == 0            # every component starts 16-byte aligned
        raw = got.contiguous().view(torch.uint8).numpy().reshape(-1) if got.numel() else np.zeros(0, np.uint8)
        assert np.array_equal(raw, np.ascontiguousarray(expect).view(np.uint8).reshape(-1))
    fmt.validate_packed(dict(container.buffers), golden.shape, container.encoded_dtype)


def test_repacking_reproduces_the_reference_blob_byte_for_byte(golden):
    container = ep.CompressedTensor.unpack(_blob(golden))
    again = pack_quant_state(container.header, container.buffers, container.shape, container.encoded_dtype)
    assert torch.equal(again, container.entropack_quant_state)
    header, start = parse_quant_state(again)
    assert start % 16 == 0 and header["buffer_names"] == list(fmt.PACKED_KEYS)


def test_state_dict_round_trip_and_sharing():
    golden = Golden("c1_256x256_bf16_3p5")
    container = ep.CompressedTensor.unpack(_blob(golden))
    state = container.state_dict()
    assert list(state) == ["entropack_quant_state"] and state["entropack_quant_state"].dtype == torch.uint8
    clone = ep.CompressedTensor.from_state_dict(state)
    assert clone.entropack_quant_state.data_ptr() == container.entropack_quant_state.data_ptr()   # shares storage
    assert ep.CompressedTensor.from_state_dict(container.state_dict("w"), "w").shape == container.shape
    with pytest.raises(ValueError):
        ep.CompressedTensor.from_state_dict({}, None)
    as_f16 = container.to(torch.float16)
    assert as_f16.dtype == torch.float16 and as_f16.encoded_dtype == torch.bfloat16
    assert as_f16.entropack_quant_state.data_ptr() == container.entropack_quant_state.data_ptr()
    independent = container.clone()
    assert independent.entropack_quant_state.data_ptr() != container.entropack_quant_state.data_ptr()
    with pytest.raises(RuntimeError):
        container.requires_grad_(True)


def test_moving_a_container_parses_nothing_and_takes_host_copies_of_its_small_tables():
    """A container that leaves the host is not parsed again (on a device that would be two read-backs), and its small
    tables keep a host copy for the decode plan. The meta device stands in for a GPU: reading a meta tensor back
    raises, so this passes only if nothing does."""
    from entropack_amd.schemes.base import HOST_MIRROR, host_copy
    golden = Golden("c1_256x256_bf16_3p5")
    container = ep.CompressedTensor.unpack(_blob(golden))
    moved = container.to("meta")
    assert moved.device.type == "meta" and moved.shape == container.shape and moved.header == container.header
    assert moved.storage_nbytes(include_header=False) == container.storage_nbytes(include_header=False)
    for name in ("layout", "stream_meta", "freq_tables", "scales"):
        assert torch.equal(host_copy(moved.buffers[name]), container.buffers[name]), name
        assert host_copy(moved.buffers[name]).data_ptr() != container.buffers[name].data_ptr()      # a copy, not a view
    assert not hasattr(container.buffers["layout"], HOST_MIRROR)                                   # host buffers need none
    big = ep.compress((torch.randn(512, 1024) * 0.02).to(torch.bfloat16), ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager"))
    assert not hasattr(big.to("meta").buffers["payload"], HOST_MIRROR)                              # only small buffers
    again = moved.clone()                                                                           # copies travel on
    assert torch.equal(host_copy(again.buffers["stream_meta"]), container.buffers["stream_meta"])


def test_torch_save_load_weights_only(tmp_path):
    golden = Golden("ragged_66x200_bf16_4p0")
    container = ep.CompressedTensor.unpack(_blob(golden))
    path = tmp_path / "ckpt.pt"
    torch.save(container.state_dict(), path)
    loaded = torch.load(path, weights_only=True)
    back = ep.CompressedTensor.from_state_dict(loaded)
    assert torch.equal(back.entropack_quant_state, container.entropack_quant_state)


def test_malformed_blobs_are_rejected():
    golden = Golden("low_64x512_bf16_2p0")
    blob = _blob(golden)
    with pytest.raises(TypeError):
        ep.CompressedTensor.unpack(blob.to(torch.int8))
    with pytest.raises(ValueError, match="too short"):
        ep.CompressedTensor.unpack(blob[:4])
    with pytest.raises(ValueError, match="truncated"):
        ep.CompressedTensor.unpack(blob[:100])
    with pytest.raises(ValueError):
        ep.CompressedTensor.unpack(blob[:-16])                                  # last buffer cut short
    with pytest.raises(ValueError, match="trailing"):
        ep.CompressedTensor.unpack(torch.cat([blob, torch.zeros(16, dtype=torch.uint8)]))
    header, _ = parse_quant_state(blob)
    container = ep.CompressedTensor.unpack(blob)
    fewer = {k: v for k, v in container.buffers.items() if k != "scales"}
    with pytest.raises(ValueError, match="must be"):
        ep.CompressedTensor({"compress_method": "lattice_rans"}, fewer, container.shape, torch.bfloat16)
    with pytest.raises(KeyError):
        ep.CompressedTensor({"compress_method": "nope"}, dict(container.buffers), container.shape, torch.bfloat16)
    garbled = blob.clone()
    garbled[8:12] = 0xFF
    with pytest.raises(ValueError, match="invalid"):
        ep.CompressedTensor.unpack(garbled)


def test_validate_packed_catches_structural_damage():
    golden = Golden("c1_256x256_bf16_3p5")
    container = ep.CompressedTensor.unpack(_blob(golden))
    good = dict(container.buffers)
    fmt.validate_packed(good, golden.shape, torch.bfloat16)
    bad = dict(good, offsets=good["offsets"].clone())
    bad["offsets"].view(torch.int32)[2] = 1
    with pytest.raises(ValueError, match="monotone"):
        fmt.validate_packed(bad, golden.shape, torch.bfloat16)
    bad = dict(good, freq_tables=good["freq_tables"].clone())
    bad["freq_tables"].view(torch.int16)[3] += 1
    with pytest.raises(ValueError, match="sum"):
        fmt.validate_packed(bad, golden.shape, torch.bfloat16)
    bad = dict(good, scales=good["scales"].clone())
    bad["scales"][5] = -1.0
    with pytest.raises(ValueError, match="positive"):
        fmt.validate_packed(bad, golden.shape, torch.bfloat16)
    with pytest.raises(ValueError, match="columns"):
        fmt.validate_packed(good, (256, 300), torch.bfloat16)


def test_config_validation():
    validate_config(ep.EntroPackLossyConfig())
    validate_config(ep.EntroPackLossyConfig(target_bpp=2, prob_bits=0, tile_elements=None))
    for bad in (dict(target_bpp=0.0), dict(target_bpp=12.0), dict(prob_bits=8), dict(tile_elements=0), dict(row_rdo_iterations=9)):
        with pytest.raises(ValueError):
            validate_config(ep.EntroPackLossyConfig(**bad))
    for bad in (dict(target_bpp="4"), dict(target_bpp=True), dict(prob_bits=11.0), dict(l2_prefetch=1), dict(row_rdo_iterations=None)):
        with pytest.raises(TypeError):
            validate_config(ep.EntroPackLossyConfig(**bad))
    assert registry.name_for_config(ep.EntroPackLossyConfig()) == "lattice_rans"
    assert registry.name_for_config(ep.RawConfig()) == "raw"
    scheme = registry.get_scheme("lattice_rans")
    with pytest.raises(TypeError, match="Unknown"):
        scheme.make_config({"bogus": 1})
    assert fmt.recommended_tile_elements(2.0) == 32768 and fmt.recommended_tile_elements(4.0) == 16384
    assert fmt.recommended_tile_elements(7.0) == 8192 and fmt.recommended_tile_elements(7.5) == 4096
    assert fmt.resolve_prob_bits(None, 7.0) == (11, True) and fmt.resolve_prob_bits(0, 7.1) == (12, True)
    assert fmt.resolve_prob_bits(13, 2.0) == (13, False)
    assert fmt.vector_tile_elements(16384) == 1820 and fmt.vector_tile_elements(100) == 32


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU behaviour")
def test_without_a_gpu_every_decode_request_fails_loudly():
    golden = Golden("zeros_16x64_bf16_4p0")
    container = ep.CompressedTensor.unpack(_blob(golden))
    reason = registry.reason("hip")
    assert reason is not None and "cuda" in reason.lower()
    with pytest.raises(ep.DispatchError) as caught:
        ep.decompress(container, ep.EntroPackLossyConfig(execution_backend="hip"))
    assert "hip" in caught.value.reasons and caught.value.scheme == "lattice_rans"
    with pytest.raises(ep.DispatchError) as caught:
        ep.decompress(container, ep.EntroPackLossyConfig(execution_backend="cuda"))
    assert caught.value.reasons == {"cuda": "not registered"}
    with pytest.raises(RuntimeError, match="no CPU decoder"):                  # auto -> eager lane -> refuses to decode
        ep.decompress(container, ep.EntroPackLossyConfig())
    assert registry.select(registry.get_scheme("lattice_rans"), None, None) == "eager"


def test_c_abi_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "entropack_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(ep_hip_[a-z0-9_]+)\s*\(", header)))
    assert declared, "no entry points found in the header"
    library = hip_backend.library()
    assert library.ep_hip_abi_version() == hip_backend.ABI_VERSION
    for name in declared:
        assert hasattr(library, name), f"{name} is declared in include/entropack_hip.h but not exported"
    assert sorted(hip_backend.EXPORTED_SYMBOLS) == declared
    assert library.ep_hip_error_string(1) == b"invalid argument"


def _describe(meta, freq, prob_bits, force=-1, lds=160 * 1024, tile_elements=16384):
    desc = hip_backend.PlanDesc()
    meta = np.ascontiguousarray(meta, dtype=np.int32)
    freq = np.ascontiguousarray(freq, dtype=np.uint16)
    status = hip_backend.library().ep_hip_plan_describe(
        meta.ctypes.data, freq.ctypes.data if freq.size else None, freq.size, prob_bits, tile_elements, lds, force, ctypes.byref(desc))
    return status, desc


def test_plan_choice_is_pure_host_logic(golden):
    prob_bits = int(golden.buffers["layout"][1])
    status, desc = _describe(golden.buffers["stream_meta"], golden.buffers["freq_tables"], prob_bits,
                             tile_elements=int(golden.buffers["layout"][2]))
    assert status == hip_backend.OK
    alphabets = golden.buffers["stream_meta"][:, 3]
    assert desc.max_alphabet == alphabets.max() and desc.alphabet_sum == alphabets.sum() and desc.prob_bits == prob_bits
    if prob_bits > 11:
        # Slot tables of 2**prob_bits entries no longer fit LDS; the rank/select form indexes the present symbols.
        assert desc.table_kind == hip_backend.TABLE_LDS_RANK
        freq = golden.buffers["freq_tables"]
        meta = golden.buffers["stream_meta"]
        present = [int(np.count_nonzero(freq[meta[s, 2]:meta[s, 2] + meta[s, 3]])) for s in range(1, 17)]
        assert list(desc.present_offset) == [0, 0] + list(np.cumsum(present))
        total = sum(present)
        rs_unit = (1 << prob_bits) // 32 * 8
        rs_at = -(-(-(-total * 4 // 16) * 16 + -(-total * 2 // 16) * 16) // rs_unit) * rs_unit
        assert desc.lds_bytes == rs_at + 16 * rs_unit and desc.table_bytes == 256 + desc.lds_bytes
        status, forced = _describe(golden.buffers["stream_meta"], golden.buffers["freq_tables"], prob_bits,
                                   force=hip_backend.TABLE_GLOBAL64)
        assert status == hip_backend.OK and forced.lds_bytes == 0 and forced.table_bytes == 256 + 17 * (1 << prob_bits) * 8
        assert not any(forced.present_offset)
    else:
        assert desc.table_kind in (hip_backend.TABLE_LDS_BYTE, hip_backend.TABLE_LDS_WIDE)
        slot_tables = 256 + 16 * (1 << prob_bits) * 4
        if desc.table_kind == hip_backend.TABLE_LDS_BYTE and prob_bits == 11:
            # 128 KiB of slot tables leave room for one workgroup per CU, so the two-level form rides along for big launches.
            assert desc.sym_offset == slot_tables and desc.table_bytes == desc.sym_offset + 16 * 256 * 8 + 16 * (1 << prob_bits)
        else:
            assert desc.sym_offset == 0 and desc.table_bytes == slot_tables
    if golden.name.startswith("huge_alpha"):
        assert desc.table_kind == hip_backend.TABLE_LDS_WIDE          # a 769-symbol alphabet cannot use byte values
    if golden.name.startswith("c1_"):
        assert desc.table_kind == hip_backend.TABLE_LDS_BYTE


def test_plan_describe_rejects_inconsistent_tables():
    golden = Golden("c1_256x256_bf16_3p5")
    meta, freq = golden.buffers["stream_meta"].copy(), golden.buffers["freq_tables"].copy()
    assert _describe(meta, freq, 11)[0] == hip_backend.OK
    assert _describe(meta, freq, 8)[0] == hip_backend.EINVAL
    broken = freq.copy()
    broken[4] += 1
    assert _describe(meta, broken, 11)[0] == hip_backend.EINVAL                # sum != 2**11
    shifted = meta.copy()
    shifted[3, 2] += 1
    assert _describe(shifted, freq, 11)[0] == hip_backend.EINVAL               # offsets not contiguous
    assert _describe(meta, freq[:-1], 11)[0] == hip_backend.EINVAL
    assert _describe(meta, freq, 11, lds=64 * 1024)[1].table_kind == hip_backend.TABLE_LDS_RANK
    # The rank/select form keeps its values in half precision while every coordinate is exact there: |z| < 1024, and
    # |m| < 512 in the last field's two streams (z7 = 2 m + parity); a minimum beyond that keeps 16-bit integers.
    assert _describe(meta, freq, 11, lds=64 * 1024)[1].rank_values_half == 1
    assert _describe(meta, freq, 11)[1].rank_values_half == 0                  # only the rank/select form has the field set
    for stream, minimum, expect in ((3, -1023, 1), (3, -1024, 0), (16, -511, 1), (16, -512, 0)):
        far = meta.copy()
        far[stream, 1] = minimum
        status, desc = _describe(far, freq, 11, force=hip_backend.TABLE_LDS_RANK)
        assert status == hip_backend.OK and desc.rank_values_half == expect, (stream, minimum)
    assert _describe(meta, freq, 11, lds=2 * 1024)[1].table_kind == hip_backend.TABLE_GLOBAL64
    assert _describe(meta, freq, 11, force=hip_backend.TABLE_GLOBAL64)[1].table_kind == hip_backend.TABLE_GLOBAL64
    assert _describe(meta, freq, 11, tile_elements=0)[0] == hip_backend.EINVAL
    # Tiles beyond 2**18 vectors are outside what the LDS-table kernels address: such plans take the global tables.
    assert _describe(meta, freq, 11, tile_elements=9 << 18)[1].table_kind == hip_backend.TABLE_LDS_BYTE
    assert _describe(meta, freq, 11, tile_elements=(9 << 18) + 9)[1].table_kind == hip_backend.TABLE_GLOBAL64
    assert _describe(meta, freq, 11, tile_elements=(9 << 18) + 9, force=hip_backend.TABLE_LDS_BYTE)[0] == hip_backend.EUNSUPPORTED
    wide_only = Golden("huge_alpha_16x1024_bf16_7p0")
    assert _describe(wide_only.buffers["stream_meta"], wide_only.buffers["freq_tables"], 11,
                     force=hip_backend.TABLE_LDS_BYTE)[0] == hip_backend.EUNSUPPORTED


def test_launch_table_form_depends_on_the_launch_size():
    """A byte-valued prob_bits-11 plan decodes small containers with its slot tables and large ones (more tile pairs
    than 16 waves on every CU hold) with its two-level section; other plans never switch. Pure host logic."""
    lib = hip_backend.library()
    golden = Golden("c1_256x256_bf16_3p5")
    _, desc = _describe(golden.buffers["stream_meta"], golden.buffers["freq_tables"], 11, tile_elements=16384)
    assert desc.table_kind == hip_backend.TABLE_LDS_BYTE and desc.sym_offset != 0
    bf16, int8, f32 = (hip_backend.STORE_KINDS[t] for t in (torch.bfloat16, torch.int8, torch.float32))
    kind = lambda d, store, rows, cols, cus=256: lib.ep_hip_decode_table_kind(ctypes.byref(d), store, rows, cols, 16384, cus)
    assert kind(desc, bf16, 256, 256) == hip_backend.TABLE_LDS_BYTE
    assert kind(desc, bf16, 8192, 28672) == hip_backend.TABLE_LDS_SYM          # 8066 pairs > 256 * 16
    assert kind(desc, int8, 8192, 28672) == hip_backend.TABLE_LDS_SYM
    assert kind(desc, f32, 8192, 28672) == hip_backend.TABLE_LDS_SYM
    assert kind(desc, bf16, 4096, 28672) == hip_backend.TABLE_LDS_BYTE         # 4033 pairs: one pass of resident waves
    assert kind(desc, bf16, 4096, 28672, 64) == hip_backend.TABLE_LDS_SYM      # ... on a quarter of the CUs it is not
    assert kind(desc, bf16, 0, 256) == -1
    _, forced = _describe(golden.buffers["stream_meta"], golden.buffers["freq_tables"], 11, force=hip_backend.TABLE_LDS_SYM)
    assert forced.table_kind == hip_backend.TABLE_LDS_SYM and kind(forced, bf16, 256, 256) == hip_backend.TABLE_LDS_SYM
    wide = Golden("huge_alpha_16x1024_bf16_7p0")
    _, wide_desc = _describe(wide.buffers["stream_meta"], wide.buffers["freq_tables"], 11)
    assert wide_desc.sym_offset == 0 and kind(wide_desc, bf16, 8192, 28672) == hip_backend.TABLE_LDS_WIDE
    assert _describe(wide.buffers["stream_meta"], wide.buffers["freq_tables"], 11, force=hip_backend.TABLE_LDS_SYM)[0] == hip_backend.EUNSUPPORTED


def test_skinny_gemm_workspace_matches_its_split():
    """Workspace = K slices x M x N x 4 bytes. A block owns 128 weight rows; slices aim at four blocks per CU, never exceed
    the 128-byte chunks of a row or 64, and are evened out."""
    size = hip_backend.library().ep_hip_gemm_skinny_workspace

    def expect(m, n, k_bytes, cus):
        rows = 128
        blocks, chunks = -(-n // rows), -(-k_bytes // 128)
        slices = max(1, min(-(-4 * cus // blocks), chunks, 64))
        per = -(-chunks // slices)
        return -(-chunks // per) * m * n * 4

    assert size(16, 8192, 28672 * 2, 256) == 16 * 16 * 8192 * 4                # 64 row blocks -> 16 slices
    assert size(1, 128, 256, 256) == 2 * 1 * 128 * 4                           # only two chunks to split
    for case in [(16, 8192, 57344, 256), (128, 8192, 57344, 256), (128, 100000, 4096, 256), (65, 300, 1 << 20, 256), (3, 77, 16, 8)]:
        assert size(*case) == expect(*case), case
    assert size(0, 10, 10, 256) == 0 and size(4, 10, 10, 0) == 0


def test_split_gemm_workspace_is_zero_unless_the_tiles_leave_half_the_cus_idle():
    """More than 128 rows: 128 x 128 tiles with K divided over the largest number of blocks per tile (at most 8, at most the
    CUs over the tiles) that leaves each a whole number of four 128-byte steps and at least eight; 0 where no such split
    exists, and 0 where 64 x 64 blocks fit the CUs in one round (one kernel then does better than two), which is how a
    caller learns that the product takes the unsplit kernels."""
    size = hip_backend.library().ep_hip_gemm_skinny_workspace

    def expect(m, n, k_bytes, cus):
        if k_bytes % 128:
            return 0
        tiles, steps = -(-m // 128) * -(-n // 128), k_bytes // 128
        small = -(-m // 64) * -(-n // 64)
        if 2 * tiles <= cus and small <= cus and steps % 4 == 0 and steps >= 8:
            return 0
        for slices in range(min(cus // tiles, 8), 1, -1):
            if steps % (4 * slices) == 0 and steps // slices >= 8:
                return slices * m * n * 4
        return 0

    assert size(384, 3072, 6144, 256) == 3 * 384 * 3072 * 4                    # 72 tiles, 48 steps: three slices of 16
    assert size(384, 3072, 2048, 256) == 2 * 384 * 3072 * 4                    # 16 steps: two slices of 8
    assert size(256, 3072, 6144, 256) == 0                                     # 192 blocks of 64 x 64 fit the CUs
    assert size(1024, 3072, 6144, 256) == 0                                    # 192 tiles: nothing to gain
    assert size(384, 3072, 6144 + 16, 256) == 0                                # K not of whole steps
    assert size(384, 3072, 512, 256) == 0                                      # four steps: too short to split
    for case in [(200, 3000, 4096, 256), (300, 1000, 2048, 256), (640, 3072, 6144, 256), (129, 128, 1 << 16, 256), (256, 3072, 6144, 64),
                 (384, 640, 8192, 304), (520, 2000, 4096, 256), (129, 4000, 2048, 256)]:
        assert size(*case) == expect(*case), case


def test_entry_points_refuse_bad_arguments_before_touching_a_device():
    """Argument checks of the C ABI run on the host: every call here must come back with EP_HIP_EINVAL (or
    EUNSUPPORTED) without a GPU in the machine. Pointers are small non-null integers that are never dereferenced."""
    import ctypes
    lib = hip_backend.library()
    EINVAL, EUNSUPPORTED = hip_backend.EINVAL, hip_backend.EUNSUPPORTED
    fake = 0x1000
    modes = (ctypes.c_uint8 * 8)(1, 0, 0, 0, 0, 0, 0, 0)

    def tile_ans(**over):
        call = dict(payload=fake, words=10, offsets=fake, states=fake, tables=fake, modes=ctypes.addressof(modes), tile=4096, pb=10, lanes=2,
                    elements=100, out=fake, error=fake)
        call.update(over)
        return lib.ep_hip_decode_tile_ans(call["payload"], call["words"], call["offsets"], call["states"], call["tables"], call["modes"],
                                          call["tile"], call["pb"], call["lanes"], call["elements"], call["out"], call["error"], None)

    assert tile_ans(offsets=None) == EINVAL and tile_ans(tables=None) == EINVAL and tile_ans(modes=None) == EINVAL
    assert tile_ans(out=None) == EINVAL and tile_ans(error=None) == EINVAL
    assert tile_ans(payload=None) == EINVAL                                    # words announced, none given
    assert tile_ans(tile=0) == EINVAL and tile_ans(elements=0) == EINVAL
    assert tile_ans(pb=8) == EINVAL and tile_ans(pb=13) == EINVAL
    assert tile_ans(lanes=3) == EINVAL and tile_ans(lanes=16) == EINVAL
    assert tile_ans(payload=fake + 1) == EINVAL                                # words are 2-byte aligned
    assert tile_ans(words=1 << 32) == EINVAL
    assert tile_ans(states=None) == EINVAL                                     # lane 1 is coded: states are needed
    bad_modes = (ctypes.c_uint8 * 8)(1, 2, 0, 0, 0, 0, 0, 0)
    assert tile_ans(modes=ctypes.addressof(bad_modes)) == EINVAL

    def rotate(**over):
        call = dict(x=fake, kind=0, rows=4, inner=256, ldx=256, group=64, codes=fake, scales=fake)
        call.update(over)
        return lib.ep_hip_rotate_quantize_rows(call["x"], call["kind"], call["rows"], call["inner"], call["ldx"], call["group"],
                                               call["codes"], call["scales"], None)

    assert rotate(x=None) == EINVAL and rotate(codes=None) == EINVAL and rotate(scales=None) == EINVAL
    assert rotate(rows=0) == EINVAL and rotate(inner=0) == EINVAL and rotate(ldx=128) == EINVAL and rotate(kind=7) == EINVAL
    for group in (0, 2, 8, 32, 100, 128):
        assert rotate(group=group) == EINVAL                                   # not a power of four
    assert rotate(inner=320, ldx=320, group=256) == EINVAL                     # does not divide the row
    assert rotate(inner=2048, ldx=2048, group=1024) == EUNSUPPORTED            # a valid group, but not one this kernel rotates
    assert rotate(x=fake + 2) == EUNSUPPORTED                                  # rows it cannot load four elements at a time
    assert lib.ep_hip_quantize_rows(None, 0, 4, 256, 256, fake, fake, None) == EINVAL


def test_static_accumulator_entry_point_checks_sizes_on_the_host():
    """ep_hip_linear_fused_bf16_static refuses what its fixed array cannot hold before it touches a device."""
    import ctypes
    lib = hip_backend.library()
    fake = 0x1000
    desc = hip_backend.PlanDesc()
    job = hip_backend.DecodeJob()
    job.desc = ctypes.pointer(desc)
    job.rows, job.cols_padded = hip_backend.STATIC_ACCUMULATOR_FLOATS // 4 + 1, 512
    call = lambda m: lib.ep_hip_linear_fused_bf16_static(ctypes.byref(job), fake, m, 512, None, fake, job.rows, 0, None)
    assert call(4) == hip_backend.ETOOLARGE
    assert call(5) == hip_backend.EUNSUPPORTED
    assert call(0) == hip_backend.EINVAL
    assert lib.ep_hip_linear_fused_bf16_static(None, fake, 1, 512, None, fake, 512, 0, None) == hip_backend.EINVAL
    assert lib.ep_hip_error_string(hip_backend.ETOOLARGE) == b"request exceeds the library's fixed scratch buffer"


def test_hip_lane_refuses_tile_sizes_the_c_abi_would_truncate():
    """`tile_elements` is an int64 in the container and a C int at the ABI: the lane must refuse what would not survive
    the conversion instead of letting the library derive different tiles than the buffers were checked against."""
    from entropack_amd.schemes.lattice_rans import hip as lane
    lane._check_abi_ranges({"tile_elements": 16384})
    lane._check_abi_ranges({"tile_elements": 2 ** 31 - 1})
    for bad in (2 ** 31, 2 ** 32 + 16384, 2 ** 40):
        with pytest.raises(ValueError, match="tile_elements"):
            lane._check_abi_ranges({"tile_elements": bad})


def test_prepared_decode_cache_keeps_no_container_alive(monkeypatch):
    """The hip lane caches a prepared call on the container's `layout` tensor. The cache must refer to the container's
    tensors weakly: dropping the container frees its payload by reference count alone, with no cycle-collector pass."""
    import contextlib
    import gc
    import types
    import weakref

    from entropack_amd.schemes.lattice_rans import hip as hip_lane

    torch.manual_seed(0)
    container = ep.compress((torch.randn(32, 64) * 0.02).to(torch.bfloat16), ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager"))
    buffers = fmt.LatticeBuffers(**{key: container.buffers[key].clone() for key in fmt.LatticeBuffers._fields})
    info = fmt.decode_geometry(buffers._asdict(), (32, 64))
    plan = hip_lane.DecodePlan(desc=hip_backend.PlanDesc(), tables=torch.zeros(256, dtype=torch.uint8), error=torch.zeros(1, dtype=torch.int32),
                               key=(0, 0, None, None))
    monkeypatch.setattr(hip_lane, "_checked_geometry", lambda *a: (info, torch.bfloat16, False))
    monkeypatch.setattr(hip_lane, "_plan_for", lambda *a: plan)
    monkeypatch.setattr(hip_lane._hip, "library", lambda: types.SimpleNamespace(ep_hip_decode_lattice=None))
    monkeypatch.setattr(torch.cuda, "device", lambda device: contextlib.nullcontext())
    monkeypatch.setattr(torch.cuda, "current_device", lambda: 0)

    prepared = hip_lane._PreparedDecode(buffers, (32, 64), torch.bfloat16)
    buffers.layout._lattice_rans_hip_calls = {(torch.bfloat16, (32, 64)): prepared}
    buffers.layout._lattice_rans_hip_plan = plan
    assert prepared.serves(buffers, (32, 64), torch.bfloat16)
    watched = [weakref.ref(tensor) for tensor in buffers]
    gc.disable()
    try:
        del buffers, prepared
        assert all(ref() is None for ref in watched)
    finally:
        gc.enable()
