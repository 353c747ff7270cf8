"""The decode launches under HIP graph capture: captured once, replayed several times with eager work and
synchronisations in between, every replay checked against the eager result. (The entry points allocate nothing, clear
nothing with memset calls and read no host memory at launch time, so a capture records plain kernel nodes.)"""
import pytest
import torch

import entropack_amd as ep

pytestmark = pytest.mark.gpu


def _fresh_like(reference):
    return [torch.zeros_like(t) for t in reference]


def test_lattice_tile_ans_and_batch_decodes_replay_from_a_graph():
    torch.manual_seed(12)
    weights = [(torch.randn(512, 1024) * 0.02).to(torch.bfloat16), (torch.randn(384, 768) * 0.03).to(torch.bfloat16),
               (torch.randn(1000, 520) * 0.01).to(torch.bfloat16)]
    lossy = [ep.compress(w, ep.EntroPackLossyConfig(target_bpp=rate, execution_backend="eager")).to("cuda")
             for w, rate in zip(weights, (4.0, 2.5, 8.0))]
    lossless = ep.compress(weights[0], ep.TileANSConfig(execution_backend="eager")).to("cuda")
    config = ep.EntroPackLossyConfig(execution_backend="hip")
    batch = ep.BatchDecompressor(lossy, config)
    arena = torch.empty(batch.arena_bytes, dtype=torch.uint8, device="cuda")

    # eager results (these calls also build the per-container plans, which read metadata back to the host once)
    expect_single = [ep.decompress(c, config) for c in lossy]
    expect_lossless = ep.decompress(lossless, ep.TileANSConfig(execution_backend="hip"))
    expect_batch = [t.clone() for t in batch(arena)]
    torch.cuda.synchronize()
    assert torch.equal(expect_lossless.cpu().view(torch.int16), weights[0].view(torch.int16))
    assert all(torch.equal(a, b) for a, b in zip(expect_single, expect_batch))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            got_single = [ep.decompress(c, config) for c in lossy]
            got_lossless = ep.decompress(lossless, ep.TileANSConfig(execution_backend="hip"))
            got_batch = batch(arena)
    torch.cuda.current_stream().wait_stream(side)

    for replay in range(4):
        for tensor in got_single + [got_lossless]:
            tensor.zero_()                                   # eager work between replays; a replay must rewrite everything
        arena.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(got_single, expect_single)), replay
        assert torch.equal(got_lossless, expect_lossless), replay
        assert all(torch.equal(a, b) for a, b in zip(got_batch, expect_batch)), replay
        scratch = torch.randn(1 << 20, device="cuda").sum()  # unrelated eager kernels and a host sync
        assert torch.isfinite(scratch).item()
    batch.check_errors()


def test_w8a8_and_bf16_layer_forwards_replay_from_a_graph():
    torch.manual_seed(3)
    dense = torch.nn.Linear(768, 512, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(512, 768) * 0.02).to(torch.bfloat16))
    layers = [ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0), forward_mode="fused").cuda(),
              ep.CompressedINT8Linear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=5.0), use_convrot=True).cuda()]
    inputs = {rows: torch.randn(rows, 768).to(torch.bfloat16).cuda() for rows in (1, 40, 300)}    # on the fly, skinny, tiled
    expect = {rows: [layer(x) for layer in layers] for rows, x in inputs.items()}
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            got = {rows: [layer(x) for layer in layers] for rows, x in inputs.items()}
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        for outs in got.values():
            for out in outs:
                out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for rows in inputs:
            bf16_out, int8_out = got[rows]
            assert torch.equal(int8_out, expect[rows][1]), (replay, rows)
            # the on-the-fly product sums with floating-point atomics: the last bit may differ from run to run
            assert torch.allclose(bf16_out.float(), expect[rows][0].float(), rtol=2e-2, atol=1e-3), (replay, rows)
            if rows > 4:
                assert torch.equal(bf16_out, expect[rows][0]), (replay, rows)
