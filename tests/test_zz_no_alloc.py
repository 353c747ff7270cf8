"""GPU parity, last part: ep_hip_linear_fused_bf16_static, the entry point that allocates nothing.

It is ep_hip_linear_fused_bf16 with the f32 accumulator in a fixed array of the library's device image instead of a
caller's workspace. Both are called through the C ABI on the same operands; the sums are added with floating-point
atomics in either, so their bf16 outputs agree up to accumulation order (the tolerance stated for linear outputs:
rel-L2 <= 1e-3, and never more than one bf16 ulp apart), and both must match F.linear on the decoded weight. Two
calls in a row, the second on a smaller weight with fewer activation rows, show that what one call leaves in the
shared array does not reach the next.
"""
import ctypes

import pytest
import torch
from torch.nn import functional as F

import entropack_amd as ep
from entropack_amd.backends import hip
from entropack_amd.schemes.lattice_rans import hip as lane

pytestmark = pytest.mark.gpu
REL_L2 = 1e-3          # tolerance stated for linear outputs (bf16 accumulate-order differences)


def _container(rows, cols, seed, bpp=4.0):
    torch.manual_seed(seed)
    weight = (torch.randn(rows, cols) * 0.02).to(torch.bfloat16)
    packed = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager")).to("cuda")
    dense = ep.decompress(packed, ep.EntroPackLossyConfig(execution_backend="hip"))
    return packed, dense


def _job(packed):
    buffers = lane.LatticeBuffers(**{name: packed.buffers[name] for name in lane.LatticeBuffers._fields})
    info, _, _ = lane._checked_geometry(buffers, tuple(packed.shape), torch.bfloat16)
    plan = lane._plan_for(buffers, info)
    return lane._job_of(buffers, info, plan, hip.STORE_KINDS[torch.bfloat16]), (buffers, plan)


def _both_entry_points(packed, dense, m_rows, seed, with_bias):
    job, keep = _job(packed)
    outer, inner = dense.shape
    torch.manual_seed(seed)
    x = torch.randn(m_rows, inner, device="cuda").to(torch.bfloat16)
    bias = (torch.randn(outer, device="cuda") * 0.01).to(torch.bfloat16) if with_bias else None
    stream = hip.current_stream(x.device)
    library = hip.library()

    with_workspace = torch.full((m_rows, outer), 7.0, dtype=torch.bfloat16, device="cuda")
    workspace = torch.empty(m_rows * outer, dtype=torch.float32, device="cuda")
    hip.check("ep_hip_linear_fused_bf16", library.ep_hip_linear_fused_bf16(
        ctypes.byref(job), x.data_ptr(), m_rows, x.stride(0), None if bias is None else bias.data_ptr(),
        with_workspace.data_ptr(), with_workspace.stride(0), hip.FLOAT_KINDS[torch.bfloat16], workspace.data_ptr(), stream))

    static = torch.full((m_rows, outer), 7.0, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    held_before = torch.cuda.memory_allocated()
    hip.check("ep_hip_linear_fused_bf16_static", library.ep_hip_linear_fused_bf16_static(
        ctypes.byref(job), x.data_ptr(), m_rows, x.stride(0), None if bias is None else bias.data_ptr(),
        static.data_ptr(), static.stride(0), hip.FLOAT_KINDS[torch.bfloat16], stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held_before
    lane.check_errors(keep[0])

    expect = F.linear(x.float(), dense.float(), None if bias is None else bias.float())
    for got in (with_workspace, static):
        error = ((got.double() - expect.to(torch.bfloat16).double()).norm() / expect.double().norm()).item()
        assert error <= REL_L2, error
    a, b = static.float(), with_workspace.float()
    floor = 1e-3 * b.pow(2).mean().sqrt()
    assert bool(((a - b).abs() <= 2.0 ** -7 * torch.maximum(torch.maximum(a.abs(), b.abs()), floor)).all())
    assert ((static.double() - with_workspace.double()).norm() / with_workspace.double().norm()).item() <= REL_L2
    return static


def test_static_accumulator_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    print("case static accumulator: 1024x2048 m=4, then 256x512 m=2, then 1024x2048 m=1", flush=True)
    big, big_dense = _container(1024, 2048, seed=41)
    small, small_dense = _container(256, 512, seed=42, bpp=3.0)
    first = _both_entry_points(big, big_dense, 4, seed=43, with_bias=True)
    second = _both_entry_points(small, small_dense, 2, seed=44, with_bias=False)      # smaller: fewer rows, fewer outputs
    third = _both_entry_points(big, big_dense, 1, seed=45, with_bias=True)
    assert first.shape == (4, 1024) and second.shape == (2, 256) and third.shape == (1, 1024)


def test_static_accumulator_entry_point_rejects_what_does_not_fit():
    packed, dense = _container(256, 512, seed=46)
    job, keep = _job(packed)
    x = torch.zeros(4, 512, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(4, 256, dtype=torch.bfloat16, device="cuda")
    library = hip.library()
    stream = hip.current_stream(x.device)
    call = lambda rows, m: library.ep_hip_linear_fused_bf16_static(
        ctypes.byref(job), x.data_ptr(), m, x.stride(0), None, y.data_ptr(), y.stride(0), hip.FLOAT_KINDS[torch.bfloat16], stream)
    assert call(256, 5) == hip.EUNSUPPORTED                       # more rows than the kernels carry
    job.rows = hip.STATIC_ACCUMULATOR_FLOATS // 4 + 1               # four rows of this many outputs pass the array's size
    assert call(job.rows, 4) == hip.ETOOLARGE
    assert library.ep_hip_error_string(hip.ETOOLARGE) == b"request exceeds the library's fixed scratch buffer"
    job.rows = 256
    assert call(256, 4) == hip.OK
    torch.cuda.synchronize()


def test_static_accumulator_entry_point_inside_a_hip_graph():
    """The entry point's advertised use: captured into a graph (kernel nodes only, nothing allocated), replayed with eager
    work in between; every replay gives the eager call's result. The library's device query has looked the accumulator's
    address up beforehand (`hip.device_info`), so the first call may already be the captured one."""
    print("case static accumulator under graph capture: 512x1024 m=3", flush=True)
    packed, dense = _container(512, 1024, seed=47)
    job, keep = _job(packed)
    hip.device_info(torch.cuda.current_device())
    library = hip.library()
    x = torch.randn(3, 1024, device="cuda").to(torch.bfloat16)
    y = torch.zeros(3, 512, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            hip.check("ep_hip_linear_fused_bf16_static", library.ep_hip_linear_fused_bf16_static(
                ctypes.byref(job), x.data_ptr(), 3, x.stride(0), None, y.data_ptr(), y.stride(0), hip.FLOAT_KINDS[torch.bfloat16],
                hip.current_stream(x.device)))
    torch.cuda.current_stream().wait_stream(side)
    expect = F.linear(x.float(), dense.float()).to(torch.bfloat16)
    for replay in range(3):
        y.zero_()
        x.copy_(torch.randn(3, 1024, device="cuda").to(torch.bfloat16))
        expect = F.linear(x.float(), dense.float())
        graph.replay()
        torch.cuda.synchronize()
        error = ((y.double() - expect.to(torch.bfloat16).double()).norm() / expect.double().norm()).item()
        assert error <= REL_L2, (replay, error)
        _ = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")       # eager work between the replays
    lane.check_errors(keep[0])
