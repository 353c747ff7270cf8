"""DecodeAhead: a layer sequence whose weights are decoded a group at a time (in line or on a second stream) must compute exactly
what the same layers compute on their own, in any call order, pass after pass."""
import pytest
import torch

import entropack_amd as ep


def make_layers(count, cls=None, mode="decode_then_gemm", rates=(4.0,), sizes=((512, 384),), seed=5):
    torch.manual_seed(seed)
    layers = []
    for index in range(count):
        rows, cols = sizes[index % len(sizes)]
        dense = torch.nn.Linear(cols, rows, dtype=torch.bfloat16)
        dense.weight.data.copy_((torch.randn(rows, cols) * 0.03).to(torch.bfloat16))
        dense.bias.data.copy_((torch.randn(rows) * 0.01).to(torch.bfloat16))
        config = ep.EntroPackLossyConfig(target_bpp=rates[index % len(rates)])
        layers.append((cls or ep.CompressedLinear).from_linear(dense, config=config, forward_mode=mode))
    return layers


def test_constructor_rejects_what_it_cannot_serve():
    layers = make_layers(2)
    with pytest.raises(ValueError, match="one GPU"):
        ep.DecodeAhead(layers)
    with pytest.raises(ValueError, match="at least one layer"):
        ep.DecodeAhead([])
    with pytest.raises(ValueError, match="group_size"):
        ep.DecodeAhead(layers, group_size=0)
    with pytest.raises(ValueError, match="lattice_rans container"):
        ep.DecodeAhead([torch.nn.Linear(4, 4)])


def chain(layers, x, order=None):
    outs = []
    for index in (order or range(len(layers))):
        outs.append(layers[index](x))
    return outs


@pytest.mark.gpu
@pytest.mark.parametrize("group_size,overlap", [(1, True), (3, True), (4, False), (16, True)])
@pytest.mark.parametrize("mode", ["decode_then_gemm", "fused"])
def test_same_outputs_as_layer_by_layer(group_size, overlap, mode):
    print("case", group_size, overlap, mode, flush=True)
    layers = [layer.cuda() for layer in make_layers(10, mode=mode, rates=(2.3, 4.0, 6.0, 8.0), sizes=((512, 384), (384, 384), (640, 384)))]
    torch.manual_seed(9)
    x = torch.randn(200, 384).to(torch.bfloat16).cuda()
    expect = chain(layers, x)
    with ep.DecodeAhead(layers, group_size=group_size, overlap=overlap) as ahead:
        assert all(layer._decode_ahead is ahead for layer in layers)
        for _ in range(3):                                         # pass after pass, the arenas are reused
            got = chain(layers, x)
            torch.cuda.synchronize()
            assert all(torch.equal(a, b) for a, b in zip(got, expect))
        order = [7, 0, 3, 3, 9, 1, 8, 2]                           # out of sequence: served all the same
        got = chain(layers, x, order)
        torch.cuda.synchronize()
        assert all(torch.equal(a, expect[index]) for a, index in zip(got, order))
        ahead.check_errors()
        assert ahead.arena_bytes >= 2 * 640 * 384
    assert all(layer._decode_ahead is None for layer in layers)
    assert all(torch.equal(a, b) for a, b in zip(chain(layers, x), expect))


@pytest.mark.gpu
def test_int8_layers_and_autograd_bypass():
    layers = [layer.cuda() for layer in make_layers(6, cls=ep.CompressedINT8Linear, rates=(4.0, 5.0))]
    torch.manual_seed(1)
    x = torch.randn(64, 384).to(torch.bfloat16).cuda()
    expect = chain(layers, x)
    ahead = ep.DecodeAhead(layers, group_size=2)
    got = chain(layers, x)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(got, expect))
    ahead.close()

    plain = [layer.cuda() for layer in make_layers(4)]
    ahead = ep.DecodeAhead(plain, group_size=2)
    probe = x.clone().requires_grad_(True)
    y = plain[0](probe)                       # autograd keeps the weight: it must not be a view of a reused arena
    for layer in plain[1:] + plain:           # later layers recycle both arenas
        layer(x)
    y.float().sum().backward()
    torch.cuda.synchronize()
    want = plain[0].dequantize("cuda").float().sum(dim=0).expand(64, 384)
    assert torch.allclose(probe.grad.float(), want, rtol=2e-2, atol=1e-3)
    with pytest.raises(ValueError, match="already attached"):
        ep.DecodeAhead(plain[:2])
    ahead.close()


@pytest.mark.gpu
def test_work_queued_before_a_recycle_keeps_its_weights():
    """Nothing synchronises between layers: products queued on the stream must have run before their arena is rewritten."""
    layers = [layer.cuda() for layer in make_layers(12, sizes=((1024, 1024),), rates=(4.0,))]
    torch.manual_seed(2)
    x = torch.randn(2048, 1024).to(torch.bfloat16).cuda()
    expect = chain(layers, x)
    torch.cuda.synchronize()
    with ep.DecodeAhead(layers, group_size=2):
        for _ in range(4):
            got = chain(layers, x)                                  # 12 layers, 6 groups, no host synchronisation inside
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(got, expect))
