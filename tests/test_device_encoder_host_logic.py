"""Host-side logic of the device encoder (no GPU): the stream statistics read from the quantise kernel's summary, the
table entries with their reciprocals, and the quantizer interface the scale search drives."""
import ctypes

import numpy as np
import pytest
import torch

from entropack_amd.schemes.lattice_rans import eager, hip_encode

INT64_MAX, INT64_MIN = np.iinfo(np.int64).max, np.iinfo(np.int64).min


def summary_of(q: eager.Quantized) -> np.ndarray:
    """What ep_hip_encode_quantize leaves for these vectors, computed from the CPU encoder's own statistics."""
    stats = q.stats()
    out = np.empty(hip_encode.SUMMARY_WORDS, dtype=np.int64)
    for k in range(16):
        n, lo, hi = stats[1 + k]
        out[2 * k], out[2 * k + 1] = (lo, hi) if n else (INT64_MAX, INT64_MIN)
    out[32] = int(q.coset.sum())
    return out


@pytest.mark.parametrize("scale", [0.2, 3.0])
def test_stats_from_the_kernel_summary_are_the_cpu_encoders(scale):
    x = torch.randn(16, 64, generator=torch.Generator().manual_seed(1))
    host = eager.HostQuantizer(x, eager.row_rms(x, x.dtype))
    q = host.quantize(scale)
    device_form = hip_encode.DeviceQuantized(torch.from_numpy(q.coset), torch.from_numpy(q.fields), summary_of(q))
    assert np.array_equal(device_form.stats(), q.stats())


def test_stats_of_one_coset_only():
    zeros = eager.HostQuantizer(torch.zeros(2, 16), torch.ones(2, 1)).quantize(1.0)
    stats = hip_encode.DeviceQuantized(torch.from_numpy(zeros.coset), torch.from_numpy(zeros.fields), summary_of(zeros)).stats()
    assert np.array_equal(stats, zeros.stats()) and stats[0].tolist() == [4, 0, 0]
    halves = eager.HostQuantizer(torch.full((2, 16), 0.5), torch.ones(2, 1)).quantize(1.0)
    stats = hip_encode.DeviceQuantized(torch.from_numpy(halves.coset), torch.from_numpy(halves.fields), summary_of(halves)).stats()
    assert np.array_equal(stats, halves.stats()) and stats[0].tolist() == [4, 0, 1] and int(stats[1, 0]) == 0


def test_quantised_vectors_put_together_from_planes_carry_the_right_summary():
    x = torch.randn(24, 64, generator=torch.Generator().manual_seed(2))
    q = eager.HostQuantizer(x, eager.row_rms(x, x.dtype)).quantize(0.4)
    coset, fields = q.planes()
    rebuilt = hip_encode.quantized_from_planes(coset.to(torch.int32), fields.clone())
    assert np.array_equal(rebuilt.stats(), q.stats())
    assert rebuilt.coset.dtype == torch.int8 and rebuilt.fields.dtype == torch.int32
    zeros = hip_encode.quantized_from_planes(torch.zeros(4, dtype=torch.int32), torch.zeros((4, 8), dtype=torch.int32))
    assert zeros.stats()[0].tolist() == [4, 0, 0] and int(zeros.stats()[2, 0]) == 0


def test_table_entries_divide_exactly():
    """state / freq from the packed reciprocal, as the kernel forms it: the high half of the product, put right once."""
    freq = np.array([1, 2, 3, 5, 7, 100, 1023, 2047, 2048, 32767, 32768], dtype=np.int64)
    cdf = np.arange(freq.size, dtype=np.int64) * 3
    packed = hip_encode.table_entries(freq, cdf).numpy().view(np.uint64)
    assert np.array_equal(packed & np.uint64(0xFFFF), freq.astype(np.uint64))
    assert np.array_equal((packed >> np.uint64(16)) & np.uint64(0xFFFF), cdf.astype(np.uint64))
    reciprocal = packed >> np.uint64(32)
    rng = np.random.default_rng(0)
    states = np.concatenate([rng.integers(1, 1 << 31, 20000), [1, 2, (1 << 31) - 1, 1 << 15, (1 << 16) - 1]]).astype(np.uint64)
    for f, r in zip(freq.astype(np.uint64), reciprocal):
        quotient = (states * r) >> np.uint64(32)
        rest = states - quotient * f
        assert np.all(rest < 2 * f)
        quotient = np.where(rest >= f, quotient + np.uint64(1), quotient)
        assert np.array_equal(quotient, states // f)


def test_device_quantizer_refuses_host_tensors():
    with pytest.raises(ValueError, match="on the GPU"):
        hip_encode.DeviceQuantizer(torch.zeros(2, 8), torch.ones(2, 1))
    with pytest.raises(ValueError, match="on the GPU"):
        hip_encode.encode(weight=torch.zeros(2, 8), target_bpp=4.0, prob_bits=None, tile_elements=16384)


def test_entry_points_refuse_bad_arguments_before_touching_a_device():
    """Argument checks come first in every encoder entry point, so they can be exercised without a GPU: null pointers,
    column counts that are no whole vectors, a scale that is not positive, misaligned buffers, tiles below 32 vectors,
    element sizes the lossless coder does not take."""
    from entropack_amd.backends import hip
    lib = hip.library()
    a = 1 << 20                                            # any 16-byte aligned non-null value: never dereferenced
    assert lib.ep_hip_encode_quantize(None, a, 64, 1.0, None, 4, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_quantize(a, a, 60, 1.0, None, 4, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_quantize(a, a, 64, 0.0, None, 4, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_quantize(a + 4, a, 64, 1.0, None, 4, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_histogram(a, a, 0, a, 8, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_histogram(a, a + 8, 16, a, 8, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_row_scales(a, a, 64, 1.0, 0, a, a, a, None, None) == hip.EINVAL
    assert lib.ep_hip_encode_row_scales(a, a, 63, 1.0, 4, a, a, a, None, None) == hip.EINVAL
    assert lib.ep_hip_encode_rans(a, a, 64, a, a, 10, 11, 31, a, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_rans(a, a, 64, a, a, 10, 16, 32, a, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_rans(a, a, 64, a + 4, a, 10, 11, 32, a, a, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_offsets(a, 0, a, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_offsets(a, 4, a, a + 4, None) == hip.EINVAL
    assert lib.ep_hip_encode_gather(a, a, 4, 0, a, None) == hip.EINVAL
    assert lib.ep_hip_encode_gather(a, a, 4, 8, a + 2, None) == hip.EINVAL            # a payload that starts on two bytes
    assert lib.ep_hip_tile_ans_histogram(a, 16, 3, a, None) == hip.EUNSUPPORTED
    assert lib.ep_hip_tile_ans_histogram(a + 1, 16, 2, a, None) == hip.EINVAL
    raw = (ctypes.c_uint8 * 2)(1, 0)
    assert lib.ep_hip_tile_ans_encode(a, 16, 2, 8, 10, a, raw, None, a, a, 8, a, None) == hip.EINVAL       # a coded lane needs states
    assert lib.ep_hip_tile_ans_encode(a, 16, 2, 8, 10, a, raw, a, a, a, 4, a, None) == hip.EINVAL          # stride below the tile
    assert lib.ep_hip_tile_ans_encode(a, 16, 5, 8, 10, a, raw, a, a, a, 8, a, None) == hip.EUNSUPPORTED


def test_both_encoder_lanes_price_with_the_cpu_lanes_size_model():
    """The device lane drives the CPU lane's scale search (`eager.resolve_scale`) and therefore its size model: coded bytes
    + 4 bytes per row + 64 (layout) + 408 (stream_meta) + 384 (slack), the constants of the reference's eager lane
    (entropack/schemes/lattice_rans/eager.py:102-107 there). The reference's CUDA lane prices without the last two
    (cuda.py:224), so a device-encoded container follows the CPU lane, not the reference's device lane; on small layers the
    settled rate differs by (408 + 384) * 8 / weights bits per weight."""
    import inspect

    from entropack_amd.schemes.lattice_rans import eager, hip_encode
    assert (eager.MODEL_LAYOUT_BYTES, eager.MODEL_STREAM_META_BYTES, eager.MODEL_SLACK_BYTES) == (64, 408, 384)
    assert "resolve_scale" in inspect.getsource(hip_encode)            # the device lane has no size model of its own
    assert "MODEL_" not in inspect.getsource(hip_encode)
