"""Batched decode: the host-side plan (no GPU) and, on the GPU, bit-equality with one-container-at-a-time decodes."""
import ctypes

import numpy as np
import pytest
import torch

import entropack_amd as ep
from entropack_amd.backends import hip as hip_backend
from conftest import Golden, golden_names


class _Launch(ctypes.Structure):
    _fields_ = [(name, ctypes.c_int) for name in
                ("table_kind", "prob_bits", "kind", "ilp", "threads", "lds_bytes", "blocks", "first_block", "pairs")]


class _Header(ctypes.Structure):
    _fields_ = [("magic", ctypes.c_uint32), ("n_jobs", ctypes.c_int), ("n_launches", ctypes.c_int), ("n_blocks", ctypes.c_int),
                ("args_offset", ctypes.c_uint64), ("blocks_offset", ctypes.c_uint64), ("total_bytes", ctypes.c_uint64),
                ("launches", _Launch * 64)]


def _host_jobs(names, compute_units=256, force=None):
    """Jobs over golden containers with made-up (aligned) device addresses: planning never dereferences them."""
    lib = hip_backend.library()
    descs, jobs, pairs = [], (hip_backend.DecodeJob * len(names))(), []
    cursor = 0
    for job, name in zip(jobs, names):
        golden = Golden(name)
        meta = np.ascontiguousarray(golden.buffers["stream_meta"], dtype=np.int32)
        freq = np.ascontiguousarray(golden.buffers["freq_tables"], dtype=np.uint16)
        cols_padded, prob_bits, tile_elements = (int(v) for v in golden.buffers["layout"])
        desc = hip_backend.PlanDesc()
        assert lib.ep_hip_plan_describe(meta.ctypes.data, freq.ctypes.data if freq.size else None, freq.size, prob_bits,
                                        tile_elements, 160 * 1024, -1 if force is None else force, ctypes.byref(desc)) == hip_backend.OK
        descs.append(desc)
        rows = golden.shape[0]
        job.payload_dev, job.payload_words = 0x10000, golden.buffers["payload"].size
        job.offsets_dev, job.states_dev, job.scales_dev, job.tables_dev, job.error_dev = 0x20000, 0x30000, 0x40000, 0x50000, 0x60000
        job.desc = ctypes.pointer(desc)
        job.out_offset = cursor
        job.store_kind = hip_backend.STORE_KINDS[getattr(torch, golden.dtype)]
        job.tile_elements, job.rows, job.cols_padded = tile_elements, rows, cols_padded
        cursor += -(-rows * cols_padded * 4 // 256) * 256
        vectors = rows * cols_padded // 8
        tile_vectors = max(32, tile_elements // 9)
        pairs.append((-(-vectors // tile_vectors) + 1) // 2)
    return jobs, descs, pairs


def _qualifies(name, force):
    """Does this golden container have the forced table form?"""
    golden = Golden(name)
    meta = np.ascontiguousarray(golden.buffers["stream_meta"], dtype=np.int32)
    freq = np.ascontiguousarray(golden.buffers["freq_tables"], dtype=np.uint16)
    _, prob_bits, tile_elements = (int(v) for v in golden.buffers["layout"])
    desc = hip_backend.PlanDesc()
    return hip_backend.library().ep_hip_plan_describe(
        meta.ctypes.data, freq.ctypes.data if freq.size else None, freq.size, prob_bits, tile_elements, 160 * 1024,
        -1 if force is None else force, ctypes.byref(desc)) == hip_backend.OK


def _plan(jobs, compute_units=256):
    lib = hip_backend.library()
    size = ctypes.c_size_t(0)
    status = lib.ep_hip_batch_plan(jobs, len(jobs), compute_units, None, ctypes.byref(size))
    if status != hip_backend.OK:
        return status, None
    blob = np.zeros(size.value, dtype=np.uint8)
    assert lib.ep_hip_batch_plan(jobs, len(jobs), compute_units, blob.ctypes.data, ctypes.byref(size)) == hip_backend.OK
    return hip_backend.OK, blob


@pytest.mark.parametrize("compute_units", [1, 8, 256])
def test_batch_plan_covers_every_pair_exactly_once(compute_units):
    names = golden_names()
    jobs, descs, pairs = _host_jobs(names)
    status, blob = _plan(jobs, compute_units)
    assert status == hip_backend.OK
    header = _Header.from_buffer_copy(blob[:ctypes.sizeof(_Header)].tobytes())
    assert header.magic == 0x45504254 and header.n_jobs == len(names) and header.total_bytes == blob.size
    assert header.args_offset % 256 == 0 and header.blocks_offset % 256 == 0
    blocks = blob[header.blocks_offset:header.blocks_offset + 16 * header.n_blocks].view(np.int32).reshape(-1, 4)
    covered = [np.zeros(p, dtype=np.int32) for p in pairs]
    seen_blocks = 0
    for launch in list(header.launches)[:header.n_launches]:
        assert launch.table_kind != hip_backend.TABLE_GLOBAL64            # every golden container has an LDS form
        assert launch.first_block == seen_blocks and launch.blocks > 0
        assert launch.threads % 64 == 0 and 64 <= launch.threads <= 1024 and launch.ilp in (1, 2)
        assert launch.lds_bytes <= 160 * 1024
        for job, first, count, _ in blocks[launch.first_block:launch.first_block + launch.blocks]:
            desc = descs[job]
            bf16 = jobs[job].store_kind == hip_backend.STORE_KINDS[torch.bfloat16]
            tables = desc.table_kind                                   # a batch always takes the two-level form where a plan has it
            if tables == hip_backend.TABLE_LDS_BYTE and desc.sym_offset:
                tables = hip_backend.TABLE_LDS_SYM
            int8 = jobs[job].store_kind == hip_backend.STORE_KINDS[torch.int8]
            assert (tables, desc.prob_bits, 13 if bf16 else 4 if int8 else -1) == (launch.table_kind, launch.prob_bits, launch.kind)
            assert count > 0 and count % 1 == 0
            covered[job][first:first + count] += 1
        seen_blocks += launch.blocks
    assert seen_blocks == header.n_blocks
    for job, marks in enumerate(covered):
        assert marks.size == pairs[job] and np.all(marks == 1), names[job]


def test_batch_plan_rejects_bad_jobs_and_short_blobs():
    lib = hip_backend.library()
    jobs, descs, _ = _host_jobs(golden_names()[:3])
    size = ctypes.c_size_t(0)
    assert lib.ep_hip_batch_plan(jobs, 0, 256, None, ctypes.byref(size)) == hip_backend.EINVAL
    assert lib.ep_hip_batch_plan(jobs, 3, 0, None, ctypes.byref(size)) == hip_backend.EINVAL
    assert lib.ep_hip_batch_plan(jobs, 3, 256, None, ctypes.byref(size)) == hip_backend.OK
    small = np.zeros(size.value - 256, dtype=np.uint8)
    short = ctypes.c_size_t(small.size)
    assert lib.ep_hip_batch_plan(jobs, 3, 256, small.ctypes.data, ctypes.byref(short)) == hip_backend.EINVAL
    jobs[1].out_offset = 8                                               # outputs are written with 16-byte stores
    assert lib.ep_hip_batch_plan(jobs, 3, 256, None, ctypes.byref(size)) == hip_backend.EINVAL
    jobs[1].out_offset = 0
    jobs[2].rows = 0
    assert lib.ep_hip_batch_plan(jobs, 3, 256, None, ctypes.byref(size)) == hip_backend.EINVAL


def test_batch_plan_gives_global64_jobs_their_own_launch():
    names = golden_names()[:4]
    jobs, descs, pairs = _host_jobs(names, force=hip_backend.TABLE_GLOBAL64)
    status, blob = _plan(jobs)
    assert status == hip_backend.OK
    header = _Header.from_buffer_copy(blob[:ctypes.sizeof(_Header)].tobytes())
    assert header.n_launches == len(names) and header.n_blocks == 0
    assert [launch.blocks for launch in list(header.launches)[:4]] == [0, 1, 2, 3]          # the job each one decodes
    assert [launch.pairs for launch in list(header.launches)[:4]] == pairs


# ---- GPU ---------------------------------------------------------------------------------------------------------------

_VIEW = {torch.bfloat16: torch.int16, torch.float16: torch.int16, torch.float32: torch.int32, torch.int8: torch.uint8}


def _bits(tensor):
    return tensor.contiguous().view(_VIEW[tensor.dtype]).cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("force", [None, hip_backend.TABLE_LDS_RANK, hip_backend.TABLE_LDS_SYM, hip_backend.TABLE_GLOBAL64],
                         ids=["auto", "lds_rank", "lds_sym", "global64"])
def test_batch_of_golden_containers_matches_reference_bits(force):
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    names = [name for name in golden_names() if _qualifies(name, force)]
    assert len(names) >= 5
    print("batch of", names, "force", force, flush=True)
    hip_lane.FORCE_TABLE_KIND = force
    try:
        containers = [ep.CompressedTensor.unpack(torch.from_numpy(Golden(name).quant_state.copy()).cuda()) for name in names]
        batch = ep.BatchDecompressor(containers, ep.EntroPackLossyConfig(execution_backend="hip"))
        first = batch()
        arena = torch.empty(batch.arena_bytes + 256, dtype=torch.uint8, device="cuda")
        arena = arena[(-arena.data_ptr()) % 256:][:batch.arena_bytes]
        second = batch(arena)                                              # same plan, caller-owned arena
    finally:
        hip_lane.FORCE_TABLE_KIND = None
    torch.cuda.synchronize()
    batch.check_errors()
    for name, a, b in zip(names, first, second):
        golden = Golden(name)
        assert a.shape == golden.shape and str(a.dtype) == "torch." + golden.dtype
        assert np.array_equal(_bits(a), golden.restored_bits), name
        assert np.array_equal(_bits(b), golden.restored_bits), name


@pytest.mark.gpu
def test_batch_of_mixed_rate_layers_equals_single_decodes():
    """A small stand-in for a transformer stack: four shapes, five rates round-robin, one pass against 20 single decodes."""
    shapes = [(384, 1152), (384, 384), (1024, 384), (384, 1024)]
    rates = [2.3, 4.0, 5.0, 6.0, 8.0]
    torch.manual_seed(3)
    containers = []
    for index in range(20):
        rows, cols = shapes[index % 4]
        weight = (torch.randn(rows, cols) * 0.02).to(torch.bfloat16)
        containers.append(ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=rates[index % 5], execution_backend="eager")).to("cuda"))
    print("mixed-rate batch of", len(containers), flush=True)
    config = ep.EntroPackLossyConfig(execution_backend="hip")
    singles = [ep.decompress(c, config) for c in containers]
    together = ep.decompress_many(containers, config)
    torch.cuda.synchronize()
    kinds = set()
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
    for container, single, batched in zip(containers, singles, together):
        lattice = LatticeBuffers(**{k: container.buffers[k] for k in LatticeBuffers._fields})
        hip_lane.check_errors(lattice)
        kinds.add(hip_lane.plan_of(lattice).table_kind)
        assert batched.shape == single.shape and batched.dtype == single.dtype
        assert torch.equal(batched.view(torch.int16), single.view(torch.int16))
    assert {"lds_byte", "lds_rank"} <= kinds                               # the batch really mixed kernel variants


@pytest.mark.gpu
def test_batch_with_a_ragged_last_slice_and_int8_codes():
    """One large container cut into many slices (the last one short) next to an int8 container."""
    torch.manual_seed(11)
    big = (torch.randn(2048, 4104) * 0.02).to(torch.bfloat16)               # 4104 = 8 * 513: odd vectors per row
    codes = torch.randint(-100, 100, (256, 512), dtype=torch.int8)
    config = ep.EntroPackLossyConfig(execution_backend="hip")
    containers = [ep.compress(big, ep.EntroPackLossyConfig(target_bpp=3.0, execution_backend="eager")).to("cuda"),
                  ep.compress(codes, ep.EntroPackLossyConfig(target_bpp=4.0, execution_backend="eager")).to("cuda")]
    print("ragged batch", flush=True)
    singles = [ep.decompress(c, config) for c in containers]
    together = ep.decompress_many(containers, config)
    torch.cuda.synchronize()
    assert torch.equal(together[0].view(torch.int16), singles[0].view(torch.int16))
    assert together[1].dtype == torch.int8 and torch.equal(together[1], singles[1])
