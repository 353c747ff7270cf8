"""GPU parity at the benchmark configurations' full sizes, where the routing differs from the small cases.

  * configuration 5, linear part: 8192 x 28672 @ 4 bpp with 1, 4, 16 and 128 activation rows in both forward modes against
    F.linear on the oracle-decoded weight, with the route each call takes asserted (multiply on the fly up to four rows,
    with the two-level tables at one row; decode + split-K product beyond);
  * the same at the two rates the configuration names, 2.0 and 8.0 bpp, whose routes differ: 2 bpp has 4033 tile pairs,
    which 16 waves on each of 256 CUs hold at once, so only a single row is multiplied on the fly (byte tables) and two to
    four rows decode first; 8 bpp needs prob_bits 12 and runs the rank/select kernels, multiplying up to four rows on the fly;
  * configuration 4 as specified: 120 layers of the four DiT shapes, rates 2.3 / 4 / 5 / 6 / 8 round-robin, one batched
    pass bit-equal to 120 single decodes and to the C oracle for every (shape, rate). The 20 distinct (shape, rate)
    containers are encoded once and each is placed on the device six times, as six layers with buffers of their own.
"""
import numpy as np
import pytest
import torch
from torch.nn import functional as F

import entropack_amd as ep
from entropack_amd.backends import hip as hip_backend
from entropack_amd.schemes.base import packed_buffers
from entropack_amd.schemes.lattice_rans import hip as hip_lane
from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
from oracle import c_oracle

pytestmark = pytest.mark.gpu
REL_L2 = 1e-3          # tolerance stated for linear outputs (bf16 accumulate-order differences)


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


def _oracle_bits(container):
    rows = container.shape[0]
    cols_padded = int(container.buffers["layout"][0])
    return c_oracle.decode(_host_arrays(container), (rows, cols_padded), "bfloat16", threads=16)


def _large_ffn_container(rate):
    """Configuration 5's weight, 8192 x 28672 bf16 N(0, 0.015) seed 4, at `rate` bpp: its container on the device and the
    oracle's decode of it."""
    torch.manual_seed(4)
    weight = (torch.randn(8192, 28672) * 0.015).to(torch.bfloat16)
    container = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=rate, execution_backend="eager"))
    del weight
    expect = torch.from_numpy(_oracle_bits(container).view(np.int16)).view(torch.bfloat16)
    return container.to("cuda"), expect.cuda()


@pytest.fixture(scope="module")
def large_ffn_weight():
    return _large_ffn_container(4.0)


def test_config_5_decode_and_small_m_linear_at_full_size(large_ffn_weight):
    on_gpu, oracle_weight = large_ffn_weight
    rows, cols = 8192, 28672
    config = ep.EntroPackLossyConfig(execution_backend="hip")
    decoded = ep.decompress(on_gpu, config)
    buffers = packed_buffers(on_gpu.buffers, LatticeBuffers)
    torch.cuda.synchronize()
    hip_lane.check_errors(buffers)
    assert torch.equal(decoded.view(torch.int16), oracle_weight.view(torch.int16))
    # 8066 tile pairs are more than 16 waves on every CU hold: the launch takes the two-level tables by itself.
    assert hip_lane.plan_of(buffers).table_kind == "lds_byte"
    assert hip_lane.launch_table_kind(buffers, shape=(rows, cols), dtype=torch.bfloat16) == "lds_sym"
    del decoded

    layers = {}
    for mode in ("decode_then_gemm", "fused", "fused_through_lds"):
        layer = ep.CompressedLinear(cols, rows, bias=False, device="cuda", dtype=torch.bfloat16, forward_mode=mode)
        layer.weight = torch.nn.Parameter(on_gpu, requires_grad=False)
        layers[mode] = layer
    reference_weight = oracle_weight.double()     # float64: the float32 library product is itself 2e-3 off for four rows of this K
    torch.manual_seed(4)
    for m in (1, 4, 16, 128):
        print("case config 5 linear, M =", m, flush=True)
        x = torch.randn(m, cols).to(torch.bfloat16).cuda()
        expect = F.linear(x.double(), reference_weight).float().to(torch.bfloat16).double()
        # The route of the fused mode: up to four rows are multiplied inside the decode kernel on a weight this large
        # (its decode is bound by throughput, and the products ride along); 16 and 128 rows are decoded and multiplied by
        # the split-K product.
        assert hip_lane.fused_linear_usable(buffers, (rows, cols), x) == (m <= 4)
        assert hip_lane.fused_linear_pays(buffers, (rows, cols), x) == (m <= 4)
        assert hip_lane.mfma_linear_usable(buffers, (rows, cols), x)
        for mode, layer in layers.items():
            before = torch.cuda.memory_allocated()
            torch.cuda.reset_peak_memory_stats()
            y = layer(x)
            torch.cuda.synchronize()
            peak = torch.cuda.max_memory_allocated()
            assert y.shape == (m, rows) and y.dtype == torch.bfloat16
            error = ((y.double() - expect).norm() / expect.norm()).item()
            assert error <= REL_L2, (mode, m, error)
            if mode == "fused_through_lds":
                # the matrix cores took the decoded tiles from LDS: nothing the size of the 470 MB dense weight was ever allocated
                assert peak - before < 64 << 20, (m, peak - before)
        if m <= 4:
            # and the multiply-on-the-fly kernel itself at this size, whatever the layer prefers
            try:
                y = hip_lane.linear_rows(buffers, shape=(rows, cols), x=x, bias=None)
            except hip_backend.HipError as error:
                assert error.status == hip_backend.EUNSUPPORTED and m > 1
            else:
                error = ((y.double() - expect).norm() / expect.norm()).item()
                assert error <= REL_L2, ("linear_rows", m, error)
    torch.cuda.synchronize()
    hip_lane.check_errors(buffers)


# rate -> (table form of the plan, table form of the full-size launch, largest M the fused mode multiplies on the fly)
CONFIG_5_ROUTES = {2.0: ("lds_byte", "lds_byte", 1), 8.0: ("lds_rank", "lds_rank", 4)}


@pytest.mark.parametrize("rate", sorted(CONFIG_5_ROUTES))
def test_config_5_small_m_linear_at_the_rates_the_configuration_names(rate):
    """Reference semantics: y = F.linear(x, decode(W)) (entropack/linear/linear.py:163-165); here against the oracle's
    decode of the same container, rel-L2 <= 1e-3, in both forward modes."""
    on_gpu, oracle_weight = _large_ffn_container(rate)
    rows, cols = 8192, 28672
    plan_kind, launch_kind, on_the_fly_up_to = CONFIG_5_ROUTES[rate]
    decoded = ep.decompress(on_gpu, ep.EntroPackLossyConfig(execution_backend="hip"))
    buffers = packed_buffers(on_gpu.buffers, LatticeBuffers)
    torch.cuda.synchronize()
    hip_lane.check_errors(buffers)
    assert torch.equal(decoded.view(torch.int16), oracle_weight.view(torch.int16))
    del decoded
    assert hip_lane.plan_of(buffers).table_kind == plan_kind
    assert hip_lane.launch_table_kind(buffers, shape=(rows, cols), dtype=torch.bfloat16) == launch_kind
    layers = {}
    for mode in ("decode_then_gemm", "fused"):
        layer = ep.CompressedLinear(cols, rows, bias=False, device="cuda", dtype=torch.bfloat16, forward_mode=mode)
        layer.weight = torch.nn.Parameter(on_gpu, requires_grad=False)
        layers[mode] = layer
    reference_weight = oracle_weight.double()     # float64: the float32 library product is itself 2e-3 off for four rows of this K
    torch.manual_seed(4)
    for m in (1, 4, 16, 128):
        print("case config 5 linear @", rate, "bpp, M =", m, flush=True)
        x = torch.randn(m, cols).to(torch.bfloat16).cuda()
        expect = F.linear(x.double(), reference_weight).float().to(torch.bfloat16).double()
        assert hip_lane.fused_linear_usable(buffers, (rows, cols), x) == (m <= 4)
        assert hip_lane.fused_linear_pays(buffers, (rows, cols), x) == (m <= on_the_fly_up_to)
        for mode, layer in layers.items():
            y = layer(x)
            assert y.shape == (m, rows) and y.dtype == torch.bfloat16
            error = ((y.double() - expect).norm() / expect.norm()).item()
            print("   ", mode, "rel-L2 vs float64 product", error, flush=True)
            assert error <= REL_L2, (rate, mode, m, error)
            if mode == "decode_then_gemm":
                # This mode is the reference's data flow, decode then torch's F.linear: the same call on the oracle's
                # weight gives the same bits.
                assert torch.equal(y, F.linear(x, oracle_weight)), (rate, mode, m)
        if m <= 4:
            # the multiply-on-the-fly kernel itself, also where the layer prefers to decode first (2 bpp, four rows)
            y = hip_lane.linear_rows(buffers, shape=(rows, cols), x=x, bias=None)
            error = ((y.double() - expect).norm() / expect.norm()).item()
            assert error <= REL_L2, (rate, "linear_rows", m, error)
    torch.cuda.synchronize()
    hip_lane.check_errors(buffers)
    del layers, on_gpu, oracle_weight, reference_weight
    torch.cuda.empty_cache()


STACK_SHAPES = ((11520, 3840), (3840, 3840), (10240, 3840), (3840, 10240))      # qkv, out, ffn-up, ffn-down as [out, in]
STACK_RATES = (2.3, 4.0, 5.0, 6.0, 8.0)


def test_config_4_all_120_layers_in_one_pass():
    torch.manual_seed(3)
    weights = [(torch.randn(rows, cols) * 0.02).to(torch.bfloat16) for rows, cols in STACK_SHAPES]
    distinct, oracle = {}, {}
    for shape_index in range(4):
        for rate_index, rate in enumerate(STACK_RATES):
            container = ep.compress(weights[shape_index], ep.EntroPackLossyConfig(target_bpp=rate, execution_backend="eager"))
            distinct[shape_index, rate_index] = container
            oracle[shape_index, rate_index] = torch.from_numpy(_oracle_bits(container).view(np.int16))
        print("encoded and oracle-decoded shape", STACK_SHAPES[shape_index], flush=True)
    del weights
    # Layer i has shape i % 4 and rate i % 5: every shape meets every rate six times in 120 layers.
    keys = [(index % 4, index % 5) for index in range(120)]
    assert all(keys.count(key) == 6 for key in distinct)
    containers = [distinct[key].to("cuda") for key in keys]
    config = ep.EntroPackLossyConfig(execution_backend="hip")
    batch = ep.BatchDecompressor(containers, config)
    together = batch()
    torch.cuda.synchronize()
    batch.check_errors()
    kinds = {}
    for index, (key, container, batched) in enumerate(zip(keys, containers, together)):
        rows, cols = STACK_SHAPES[key[0]]
        assert batched.shape == (rows, cols) and batched.dtype == torch.bfloat16
        single = ep.decompress(container, config)
        assert torch.equal(batched.view(torch.int16), single.view(torch.int16)), index
        del single
        if index < 20:                                            # the first 20 layers are the 20 (shape, rate) pairs
            assert torch.equal(batched.view(torch.int16).cpu(), oracle[key]), key
        lattice = packed_buffers(container.buffers, LatticeBuffers)
        kind = hip_lane.plan_of(lattice).table_kind
        kinds[kind] = kinds.get(kind, 0) + 1
    torch.cuda.synchronize()
    # 8 bpp (every fifth layer) needs prob_bits 12 and the rank/select tables; the other rates are byte-valued.
    assert kinds == {"lds_byte": 96, "lds_rank": 24}, kinds
