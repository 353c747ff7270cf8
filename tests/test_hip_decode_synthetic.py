"""GPU parity, part 2: containers made by this package's encoder (bit-identical to the reference's on the golden set),
decoded by the HIP lane and checked bit for bit against the CPU oracle, from 8-column slivers up to 8192 x 28672."""
import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.backends import hip as hip_backend
from entropack_amd.schemes.lattice_rans import hip as hip_lane
from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
from oracle import c_oracle

pytestmark = pytest.mark.gpu


def host_buffers(container):
    out = {}
    for key, value in container.buffers.items():
        value = value.detach().cpu()
        if value.dtype == torch.uint16:
            out[key] = value.view(torch.int16).numpy().view(np.uint16)
        elif value.dtype == torch.uint32:
            out[key] = value.view(torch.int32).numpy().view(np.uint32)
        else:
            out[key] = value.numpy()
    return out


def gauss(seed, rows, cols, sigma=0.02, outliers=False):
    torch.manual_seed(seed)
    weight = torch.randn(rows, cols) * sigma
    if outliers:
        index = torch.randperm(rows * cols)[: int(round(rows * cols * 0.001))]
        weight.view(-1)[index] *= 20.0
    return weight.to(torch.bfloat16)


def decode_and_check(weight, kinds=(None,), dtype=torch.bfloat16, **options):
    container = ep.compress(weight, ep.EntroPackLossyConfig(execution_backend="eager", **options))
    assert container.compress_method == "lattice_rans"
    rows, cols = weight.shape
    padded = int(container.buffers["layout"][0])
    name = str(dtype).removeprefix("torch.")
    expect = c_oracle.decode(host_buffers(container), (rows, padded), name, threads=8)[:, :cols]
    on_gpu = container.to("cuda")
    used = []
    for kind in kinds:
        hip_lane.FORCE_TABLE_KIND = kind
        try:
            restored = ep.decompress(on_gpu.to(dtype) if dtype != weight.dtype else on_gpu, ep.EntroPackLossyConfig(execution_backend="hip"))
        except hip_backend.HipError as error:
            if error.status == hip_backend.EUNSUPPORTED:
                continue
            raise
        finally:
            hip_lane.FORCE_TABLE_KIND = None
        torch.cuda.synchronize()
        lattice = LatticeBuffers(**{k: on_gpu.buffers[k] for k in LatticeBuffers._fields})
        hip_lane.check_errors(lattice)
        used.append(hip_lane.plan_of(lattice).table_kind)
        assert restored.shape == (rows, cols) and restored.dtype == dtype
        if dtype == torch.bfloat16:
            got = restored.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        else:
            got = restored.cpu().numpy()
        assert np.array_equal(got, expect), f"kind {kind}"
    assert used
    return container, used


ALL_KINDS = (None, hip_backend.TABLE_GLOBAL64, hip_backend.TABLE_LDS_BYTE, hip_backend.TABLE_LDS_WIDE, hip_backend.TABLE_LDS_RANK,
             hip_backend.TABLE_LDS_SYM)


def test_config_2_outliers_4096x4096():
    """Benchmark configuration 2: 4096x4096, 0.1 % of entries x20, seed 1, 4.0 bpp; bit-exact against the oracle."""
    container, used = decode_and_check(gauss(1, 4096, 4096, outliers=True), kinds=ALL_KINDS, target_bpp=4.0)
    assert "lds_wide" in used and "global64" in used        # the outliers push the alphabets past a byte
    assert 4.0 < container.actual_bpp < 4.25


@pytest.mark.parametrize("bpp", [2.3, 4.0, 5.0, 6.0, 8.0])
def test_dit_like_layer_at_each_rate(bpp):
    """Benchmark configuration 4, one representative of each rate on the out-projection shape (3840 x 3840), seed 3."""
    print("case bpp", bpp, flush=True)
    container, used = decode_and_check(gauss(3, 3840, 3840), kinds=(None, hip_backend.TABLE_GLOBAL64), target_bpp=bpp)
    assert abs(container.actual_bpp - bpp) < 0.12
    assert used[0] == ("lds_rank" if bpp > 7.0 else "lds_byte")
    if bpp > 7.0:
        # Values this small are exact in half precision: the rank/select tables hold the coordinates in that form.
        on_gpu = container.to("cuda")
        ep.decompress(on_gpu, ep.EntroPackLossyConfig(execution_backend="hip"))
        lattice = LatticeBuffers(**{k: on_gpu.buffers[k] for k in LatticeBuffers._fields})
        assert hip_lane.plan_of(lattice).desc.rank_values_half == 1


def test_rank_tables_with_values_beyond_half_precision():
    """One column a thousand times the rest: alphabets thousands of values wide with few of them present. The rank/select
    tables then keep 16-bit integers (z + 1/2 is not exact in half precision beyond 1023) and the kernel its integer
    reconstruction; the general kernel decodes the same container too."""
    torch.manual_seed(26)
    weight = torch.randn(32, 32768) * 0.02
    weight[:, 100] *= 1000.0
    container, used = decode_and_check(weight.to(torch.bfloat16), kinds=(hip_backend.TABLE_LDS_RANK, None, hip_backend.TABLE_GLOBAL64), target_bpp=4.0)
    assert used[0] == "lds_rank"
    on_gpu = container.to("cuda")
    hip_lane.FORCE_TABLE_KIND = hip_backend.TABLE_LDS_RANK
    try:
        ep.decompress(on_gpu, ep.EntroPackLossyConfig(execution_backend="hip"))
    finally:
        hip_lane.FORCE_TABLE_KIND = None
    lattice = LatticeBuffers(**{k: on_gpu.buffers[k] for k in LatticeBuffers._fields})
    plan = hip_lane.plan_of(lattice)
    assert plan.table_kind == "lds_rank" and plan.desc.rank_values_half == 0
    meta = container.buffers["stream_meta"]
    assert int(meta[1:, 1].min()) < -1023 or int((meta[1:, 1] + meta[1:, 3]).max()) > 1024


@pytest.mark.parametrize("shape", [(3840, 11520), (10240, 3840)])
def test_dit_like_wide_and_tall_shapes(shape):
    decode_and_check(gauss(3, *shape), target_bpp=4.0)


@pytest.mark.parametrize("shape", [(1, 8), (3, 8), (1000, 8), (5, 16), (7, 200), (33, 1001), (2, 29120), (64, 14560), (1, 232960),
                                   (20000, 8), (5000, 40), (700, 264)])
def test_edge_shapes(shape):
    """One-vector rows, padded columns, single short tile, rows that are exactly one or sixteen tiles long; full tiles
    whose 32-vector groups span many rows (rows of 1, 5 and 33 vectors)."""
    print("case", shape, flush=True)
    decode_and_check(gauss(21, *shape, sigma=1.0), kinds=ALL_KINDS, target_bpp=4.0)


@pytest.mark.parametrize("options", [dict(target_bpp=1.0), dict(target_bpp=0.3), dict(target_bpp=6.9), dict(target_bpp=4.0, prob_bits=9),
                                     dict(target_bpp=3.0, prob_bits=10), dict(target_bpp=5.0, prob_bits=14), dict(target_bpp=4.0, tile_elements=288),
                                     dict(target_bpp=4.0, tile_elements=100000), dict(target_bpp=10.5)])
def test_rates_precisions_and_tile_sizes(options):
    print("case", options, flush=True)
    decode_and_check(gauss(22, 512, 1024), kinds=ALL_KINDS, **options)


def test_tiles_beyond_the_lds_kernels_take_the_global_tables():
    """A tile of more than 2**18 vectors is outside what the LDS-table kernels address; its plan picks the general
    kernel by itself, and forcing an LDS form is refused rather than run."""
    container, used = decode_and_check(gauss(24, 640, 4096), kinds=(None, hip_backend.TABLE_LDS_BYTE), target_bpp=4.0,
                                       tile_elements=(9 << 18) + 9)
    assert used == ["global64"]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16, torch.int8])
def test_rows_with_unusual_scales_take_the_literal_formula(dtype):
    """Row scales that are zero, negative, subnormal, tiny or near the top of the float range (no encoder makes them,
    a container may hold them) must give the reference's (z + c / 2) * scale, then its container cast, bit for bit:
    the kernels' fused multiply-add is only used for ordinary scales. Ordinary and unusual rows alternate, so both
    forms run inside one tile, in whole groups and in a tile's short first group."""
    container = ep.compress(gauss(25, 96, 512), ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager"))
    odd = [0.0, -0.0, -0.02, 1e-41, 3e-39, 1e-31, 9e-31, 2e30, 7e36, 3e38, -3e38]
    scales = container.buffers["scales"].clone()
    for row in range(0, scales.numel(), 2):
        scales[row] = odd[(row // 2) % len(odd)]
    buffers = dict(container.buffers)
    buffers["scales"] = scales
    host = host_buffers(container)
    host["scales"] = scales.numpy()
    name = str(dtype).removeprefix("torch.")
    expect = c_oracle.decode(host, (96, 512), name, threads=4)
    for kind in ALL_KINDS:
        hip_lane.FORCE_TABLE_KIND = kind
        try:
            lattice = LatticeBuffers(**{k: v.cuda() for k, v in buffers.items()})
            got = hip_lane.decode(lattice, shape=(96, 512), dtype=dtype)
        except hip_backend.HipError as error:
            if error.status == hip_backend.EUNSUPPORTED:
                continue
            raise
        finally:
            hip_lane.FORCE_TABLE_KIND = None
        torch.cuda.synchronize()
        hip_lane.check_errors(lattice)
        if dtype in (torch.bfloat16, torch.float16):                 # the oracle returns their bit patterns
            got, reference = got.view(torch.int16).cpu().numpy().view(np.uint16), expect
        elif dtype == torch.float32:
            got, reference = got.cpu().numpy().view(np.int32), expect.view(np.int32)
        else:
            got, reference = got.cpu().numpy(), expect
        assert np.array_equal(got, reference), f"kind {kind}"


def test_constant_and_zero_tensors():
    decode_and_check(torch.zeros(64, 256, dtype=torch.bfloat16), kinds=ALL_KINDS, target_bpp=4.0)
    decode_and_check(torch.full((64, 256), 0.5, dtype=torch.bfloat16), kinds=ALL_KINDS, target_bpp=4.0)
    sparse = torch.zeros(128, 512, dtype=torch.bfloat16)
    sparse[::7, ::5] = 1.0
    decode_and_check(sparse, kinds=ALL_KINDS, target_bpp=2.0)


def test_int8_code_container_decodes_to_int8():
    torch.manual_seed(23)
    weight = torch.randn(1024, 2048) * 0.02
    scale = weight.abs().amax(dim=1) / 127.0
    codes = (weight / scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)
    decode_and_check(codes, kinds=ALL_KINDS, dtype=torch.int8, target_bpp=4.0)


def test_full_size_target_8192x28672():
    """The headline shape at 2.0, 4.0 and 8.0 bpp (Benchmark configuration 5 + the 4 bpp target): bit-exact against the oracle,
    decode is idempotent, and no tile reports an error."""
    weight = gauss(4, 8192, 28672, sigma=0.015)
    for bpp in (4.0, 2.0, 8.0):
        print("case bpp", bpp, flush=True)
        container, used = decode_and_check(weight, target_bpp=bpp)
        assert abs(container.actual_bpp - bpp) < 0.1
        on_gpu = container.to("cuda")
        first = ep.decompress(on_gpu, ep.EntroPackLossyConfig(execution_backend="hip"))
        second = ep.decompress(on_gpu, ep.EntroPackLossyConfig())          # "auto" resolves to hip on this box
        assert torch.equal(first, second)
        lattice = LatticeBuffers(**{k: on_gpu.buffers[k] for k in LatticeBuffers._fields})
        # Byte plans at prob_bits 11 switch to their two-level section when the launch has more tile pairs than 16 waves
        # per CU hold (8066 at 4 bpp; the 4033 pairs at 2 bpp are one pass and stay); prob_bits 12 uses rank/select.
        expected = {2.0: "lds_byte", 4.0: "lds_sym", 8.0: "lds_rank"}[bpp]
        assert hip_lane.launch_table_kind(lattice, shape=(8192, 28672), dtype=torch.bfloat16) == expected
        del first, second, on_gpu, container
        torch.cuda.empty_cache()
