"""GPU parity, part 3: the MFMA GEMMs, the row quantiser and the compressed linear layers."""
import io

import numpy as np
import pytest
import torch
from torch.nn import functional as F

import entropack_amd as ep
from entropack_amd.linear import kernels

pytestmark = pytest.mark.gpu
REL_L2 = 1e-3          # tolerance stated for linear outputs (bf16 accumulate-order differences)


def rel_l2(got, expect):
    """Relative L2 distance. A bf16 result is compared with the fp32 reference rounded to bf16 once, which is what the
    reference layer returns; what is left is accumulation-order noise (a final-ulp flip here and there)."""
    if got.dtype == torch.bfloat16 and expect.dtype == torch.float32:
        expect = expect.to(torch.bfloat16)
    got, expect = got.double(), expect.double()
    return ((got - expect).norm() / expect.norm().clamp_min(1e-30)).item()


def within_one_ulp(got, rounded):
    """|got - rounded| <= one bf16 ulp of the larger magnitude (values that cancel to ~0 get the output's rms as floor)."""
    a, b = got.float(), rounded.float()
    floor = 1e-3 * b.pow(2).mean().sqrt()
    return bool(((a - b).abs() <= 2.0 ** -7 * torch.maximum(torch.maximum(a.abs(), b.abs()), floor)).all())


@pytest.mark.parametrize("shape", [(4096, 3072, 3072), (1, 256, 512), (17, 100, 72), (130, 129, 264), (128, 8192, 1024),
                                   (5, 300, 1000), (64, 257, 4104), (100, 128, 128), (33, 1000, 28672), (96, 640, 8),
                                   (4100, 4200, 520),           # 17 x 17 ragged 256 x 256 block tiles
                                   (4096, 3072, 256), (4096, 3000, 264),    # 256 x 192 block tiles, whole and ragged
                                   (4096, 4096, 448), (4096, 3072, 64), (4096, 3072, 192),    # whole 256 x 256 tiles; 1 and 3 K steps
                                   (768, 3072, 320), (3072, 3000, 264), (512, 3072, 128),     # 48 whole tiles; 192 ragged ones; too few
                                   (256, 256, 64), (384, 640, 192), (1024, 3072, 320),        # whole 128 x 128 tiles
                                   (300, 1000, 1024), (130, 136, 64), (1000, 3000, 320), (300, 1001, 128),   # overhanging ones
                                   (3000, 3100, 192),                                           # overhanging 256 x 192 tiles
                                   (256, 3072, 3072), (1024, 3072, 1024), (640, 3072, 256),    # one 128 x 128 tile per CU at most and
                                   (200, 3000, 2048),                                           # K of 4n steps: the four-stage kernel
                                   (384, 3072, 1024), (520, 2000, 2048), (129, 4000, 1024),     # ... with K split over blocks
                                   (900, 2900, 1024), (640, 3072, 2048)])                        # ... with 128 x 96 blocks
@pytest.mark.parametrize("with_bias", [True, False])
def test_gemm_bf16_matches_fp32_matmul(shape, with_bias):
    print("case", shape, with_bias, flush=True)
    m, n, k = shape
    torch.manual_seed(5)
    x = torch.randn(m, k, device="cuda").to(torch.bfloat16)
    w = (torch.randn(n, k, device="cuda") * 0.02).to(torch.bfloat16)
    b = (torch.randn(n, device="cuda") * 0.01).to(torch.bfloat16) if with_bias else None
    got = kernels.gemm_bf16(x, w, b)
    expect = x.float() @ w.float().T + (b.float() if with_bias else 0.0)
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    # One bf16 rounding of an f32-accumulated sum: equal to bf16(fp32 reference) except where accumulation order
    # moves a value across a rounding boundary, and then off by exactly one bf16 ulp.
    rounded = expect.to(torch.bfloat16)
    flipped = got != rounded
    assert flipped.float().mean().item() < 0.01
    assert within_one_ulp(got, rounded)
    if got.numel() >= 100000:                         # on small outputs a single flip already exceeds 1e-3
        assert rel_l2(got, expect) <= REL_L2
    as_f32 = kernels.gemm_bf16(x, w, b, out_dtype=torch.float32)
    assert rel_l2(as_f32, expect) <= 1e-5
    # Every output kind is one rounding of the same f32 sums, whichever way the kernel's epilogue writes them out.
    assert torch.equal(got, as_f32.to(torch.bfloat16))
    half_bias = None if b is None else b.to(torch.float16)
    as_f16 = kernels.gemm_bf16(x, w, half_bias, out_dtype=torch.float16)
    assert torch.equal(as_f16, kernels.gemm_bf16(x, w, half_bias, out_dtype=torch.float32).to(torch.float16))


def test_gemm_on_randomly_drawn_shapes_of_every_tile_family():
    """60 bf16 and 40 int8 products from a fixed seed, drawn so that every kernel family and the boundaries between them come up
    (few tiles, one round of 128-row blocks, several rounds, 256-row tiles, K of whole and of ragged tile steps, overhanging M
    and N): bf16 within one ulp of the f32 product rounded once, int8 exact."""
    rng = np.random.default_rng(77)
    for draw in range(100):
        int8 = draw >= 60
        m = int(rng.choice([rng.integers(129, 700), rng.integers(700, 2600), rng.integers(2600, 5000), 128 * rng.integers(2, 33)]))
        n = int(rng.choice([rng.integers(8, 700), rng.integers(700, 4200), 64 * rng.integers(1, 60), 96 * rng.integers(1, 40)]))
        step = 128 if int8 else 64
        k = int(rng.choice([step * rng.integers(1, 40), 4 * step * rng.integers(1, 12), (16 if int8 else 8) * rng.integers(1, 300)]))
        print("draw", draw, "int8" if int8 else "bf16", (m, n, k), flush=True)
        torch.manual_seed(draw)
        if int8:
            a = torch.randint(-127, 128, (m, k), device="cuda", dtype=torch.int8)
            b = torch.randint(-127, 128, (n, k), device="cuda", dtype=torch.int8)
            sa = torch.rand(m, device="cuda") * 0.05 + 1e-3
            sb = torch.rand(n, device="cuda") * 0.01 + 1e-4
            exact = a.double() @ b.double().T
            expect = exact.float() * sa.unsqueeze(1) * sb.unsqueeze(0)
            assert torch.equal(kernels.int8_gemm(a, b, sa, sb, None, torch.float32), expect), (m, n, k)
        else:
            x = torch.randn(m, k, device="cuda").to(torch.bfloat16)
            w = (torch.randn(n, k, device="cuda") * 0.02).to(torch.bfloat16)
            got = kernels.gemm_bf16(x, w, None)
            expect = x.float() @ w.float().T
            assert within_one_ulp(got, expect.to(torch.bfloat16)), (m, n, k)
            assert rel_l2(kernels.gemm_bf16(x, w, None, out_dtype=torch.float32), expect) <= 1e-5, (m, n, k)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gemm_output_rows_that_are_not_16_byte_aligned(out_dtype):
    """The 256-row kernel stores whole row pieces of 16 bytes when the output allows it; an output whose rows do not
    start on 16-byte boundaries (here: a view with an odd row stride) takes the element-wise stores and must give the
    same bits."""
    from entropack_amd.backends import hip
    m, n, k = 4096, 3072, 256
    torch.manual_seed(6)
    x = torch.randn(m, k, device="cuda").to(torch.bfloat16)
    w = (torch.randn(n, k, device="cuda") * 0.02).to(torch.bfloat16)
    bias = (torch.randn(n, device="cuda") * 0.01).to(out_dtype)
    expect = kernels.gemm_bf16(x, w, bias, out_dtype=out_dtype)
    padded = torch.full((m, n + 1), 7.0, dtype=out_dtype, device="cuda")
    hip.check("ep_hip_gemm_bf16", hip.library().ep_hip_gemm_bf16(
        x.data_ptr(), w.data_ptr(), bias.data_ptr(), padded.data_ptr(), m, n, k, x.stride(0), w.stride(0), padded.stride(0),
        hip.FLOAT_KINDS[out_dtype], hip.current_stream(x.device)))
    torch.cuda.synchronize()
    assert torch.equal(padded[:, :n], expect)
    assert bool((padded[:, n] == 7.0).all())


def test_gemm_bf16_takes_strided_rows_and_batches():
    torch.manual_seed(6)
    big = torch.randn(64, 512, device="cuda").to(torch.bfloat16)
    x = big[:, :256]                                   # row stride 512, 256 used
    w = (torch.randn(96, 256, device="cuda") * 0.1).to(torch.bfloat16)
    assert rel_l2(kernels.gemm_bf16(x, w, None, out_dtype=torch.float32), x.float() @ w.float().T) <= 1e-5
    batched = torch.randn(3, 5, 256, device="cuda").to(torch.bfloat16)
    out = kernels.gemm_bf16(batched, w, None, out_dtype=torch.float32)
    assert out.shape == (3, 5, 96)
    assert rel_l2(out, batched.float() @ w.float().T) <= 1e-5
    with pytest.raises(TypeError):
        kernels.gemm_bf16(x.float(), w, None)
    with pytest.raises(ValueError):
        kernels.gemm_bf16(x, w[:, :128], None)


@pytest.mark.parametrize("rows,inner,dtype", [(4096, 3072, torch.bfloat16), (3, 1000, torch.float32), (1, 8, torch.float16), (257, 4100, torch.bfloat16)])
def test_quantize_rows_is_exact(rows, inner, dtype):
    torch.manual_seed(7)
    x = (torch.randn(rows, inner, device="cuda") * 3).to(dtype)
    x[0, :] = 0                                        # an all-zero row takes the epsilon scale
    codes, scale = kernels.quantize_rows(x)
    # IEEE float32 arithmetic, evaluated on the CPU (torch's GPU division by a Python scalar multiplies by a
    # reciprocal instead, which is neither this definition nor the reference kernel's)
    flat = x.float().cpu()
    expect_scale = (flat.abs().amax(dim=1) / torch.tensor(127.0)).clamp(min=torch.finfo(torch.float32).eps)
    expect_codes = (flat / expect_scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)
    assert torch.equal(scale.cpu(), expect_scale)
    assert torch.equal(codes.cpu(), expect_codes)
    assert codes[0].abs().max() == 0


def test_quantize_rows_is_exact_next_to_rounding_boundaries():
    """Quotients within a few units in the last place of k + 1/2, on both sides, for scales that are not powers of
    two: where multiplying by a reciprocal and dividing can round to different integers. The kernel must give the
    division's answer everywhere."""
    torch.manual_seed(17)
    rows, inner = 64, 2048
    top = (torch.rand(rows, dtype=torch.float64) * 900 + 0.37)                      # row maxima, so scale = top / 127
    scale = (top.float() / torch.tensor(127.0)).double()
    k = torch.randint(-126, 126, (rows, inner)).double() + 0.5
    nudge = torch.randint(-3, 4, (rows, inner)).double() * 2.0 ** -23                  # relative: a few ulps either way
    x = (k * scale.unsqueeze(1) * (1.0 + nudge)).float()
    x[:, 0] = top.float()                                                              # pins each row's maximum
    x = x.cuda()
    codes, got_scale = kernels.quantize_rows(x)
    flat = x.cpu()
    expect_scale = (flat.abs().amax(dim=1) / torch.tensor(127.0)).clamp(min=torch.finfo(torch.float32).eps)
    expect_codes = (flat / expect_scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)
    assert torch.equal(got_scale.cpu(), expect_scale)
    assert torch.equal(codes.cpu(), expect_codes)
    # the construction does what it says: a reciprocal multiply alone gets some of these wrong
    naive = (flat * (1.0 / expect_scale).unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)
    assert (naive != expect_codes).any()


@pytest.mark.parametrize("shape", [(4096, 3072, 3072), (5, 70, 48), (129, 130, 1040), (4100, 4200, 528), (1, 300, 4112), (128, 1000, 28672),
                                   (33, 257, 16), (4096, 3000, 272), (4096, 4096, 896), (4096, 3072, 128), (4096, 3072, 384),
                                   (768, 3072, 640), (3072, 3000, 272), (256, 128, 128), (384, 640, 384), (1024, 3072, 640),
                                   (300, 1000, 1024), (130, 129, 128), (3000, 3100, 256),
                                   (256, 3072, 3072), (1024, 3072, 512), (200, 3000, 4096),     # the four-stage kernel, whole and ragged
                                   (384, 3072, 2048), (520, 2000, 4096),                         # ... with K split over blocks
                                   (900, 2900, 2048)])                                           # ... with 128 x 96 blocks
def test_int8_gemm_is_exact_in_f32_and_rounds_once(shape):
    print("case", shape, flush=True)
    m, n, k = shape
    torch.manual_seed(8)
    a = torch.randint(-127, 128, (m, k), device="cuda", dtype=torch.int8)
    b = torch.randint(-127, 128, (n, k), device="cuda", dtype=torch.int8)
    sa = torch.rand(m, device="cuda") * 0.05 + 1e-3
    sb = torch.rand(n, device="cuda") * 0.01 + 1e-4
    bias = (torch.randn(n, device="cuda") * 0.01).to(torch.bfloat16)
    exact = (a.double() @ b.double().T)                # |sum| < 2^31 here, exact in float64
    assert exact.abs().max() < 2 ** 31
    product = exact.float()                             # int32 -> f32 conversion (round to nearest), as the kernel does
    expect = product * sa.unsqueeze(1) * sb.unsqueeze(0)
    got = kernels.int8_gemm(a, b, sa, sb, None, torch.float32)
    assert torch.equal(got, expect)
    with_bias = kernels.int8_gemm(a, b, sa, sb, bias.float(), torch.float32)
    assert torch.equal(with_bias, expect + bias.float().unsqueeze(0))
    as_bf16 = kernels.int8_gemm(a, b, sa, sb, bias, torch.bfloat16)
    assert torch.equal(as_bf16, (expect + bias.float().unsqueeze(0)).to(torch.bfloat16))


def _c3_layer(mode, rows=3072, cols=3072, cls=None, bpp=4.0):
    torch.manual_seed(2)
    weight = (torch.randn(rows, cols) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(rows) * 0.01).to(torch.bfloat16)
    dense = torch.nn.Linear(cols, rows, dtype=torch.bfloat16)
    dense.weight.data.copy_(weight)
    dense.bias.data.copy_(bias)
    cls = cls or ep.CompressedLinear
    layer = cls.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=bpp), forward_mode=mode)
    return layer.to("cuda"), weight, bias


@pytest.mark.parametrize("mode", ["decode_then_gemm", "fused"])
def test_compressed_linear_forward_config_3(mode):
    """Benchmark configuration 3: W 3072x3072 @ 4 bpp, bias, X [4096, 3072]; output rel-L2 vs F.linear(x, W_dec, b) <= 1e-3."""
    layer, weight, bias = _c3_layer(mode)
    torch.manual_seed(2)
    x = torch.randn(4096, 3072).to(torch.bfloat16).cuda()
    y = layer(x)
    decoded = layer.dequantize("cuda")
    assert decoded.dtype == torch.bfloat16 and decoded.shape == (3072, 3072)
    expect = F.linear(x.float(), decoded.float(), bias.cuda().float())
    assert y.shape == (4096, 3072) and y.dtype == torch.bfloat16
    assert rel_l2(y, expect) <= REL_L2
    assert 0.05 < rel_l2(decoded.cpu().float(), weight.float()) < 0.09     # ~7 % at 4 bpp (E8 high-rate closed form 6.9 %)
    assert 3.9 < layer.compressed_bits < 4.1


@pytest.mark.parametrize("m", [256, 1024, 4096])
def test_fused_mode_with_this_librarys_tiled_product(m, monkeypatch):
    """`fused.TILED_PRODUCT = "own"`: more than 128 rows are multiplied by this library's kernels (blocks of 64 x 64 at 256 rows,
    of 128 x 96 at 1024, of 256 x 192 at 4096) and the vendor library is not called. The default, "auto", does the same at 256
    rows and calls the library at 4096."""
    from entropack_amd.linear import fused as fused_mode
    print("case own tiled product, M =", m, flush=True)
    layer, _, bias = _c3_layer("fused")
    torch.manual_seed(12)
    x = torch.randn(m, 3072).to(torch.bfloat16).cuda()
    decoded = layer.dequantize("cuda")
    expect = F.linear(x.float(), decoded.float(), bias.cuda().float())
    monkeypatch.setattr(fused_mode, "TILED_PRODUCT", "own")

    def no_library(*args, **kwargs):
        raise AssertionError("the vendor product was called")

    monkeypatch.setattr(fused_mode.F, "linear", no_library)
    y = layer(x)
    monkeypatch.setattr(fused_mode, "TILED_PRODUCT", "auto")
    if m == 256:
        assert torch.equal(layer(x), y)
    elif m == 4096:
        with pytest.raises(AssertionError, match="vendor product"):
            layer(x)
    monkeypatch.undo()
    assert y.shape == (m, 3072) and y.dtype == torch.bfloat16
    assert rel_l2(y, expect) <= REL_L2
    assert within_one_ulp(y, expect.to(torch.bfloat16))


@pytest.mark.parametrize("m", [1, 16, 128])
def test_compressed_linear_small_m_both_modes_agree(m):
    layer_a, _, bias = _c3_layer("decode_then_gemm", rows=512, cols=2048)
    layer_b, _, _ = _c3_layer("fused", rows=512, cols=2048)
    torch.manual_seed(9)
    x = torch.randn(2, m, 2048).to(torch.bfloat16).cuda()
    expect = F.linear(x.float(), layer_a.dequantize("cuda").float(), bias.cuda().float())
    for layer in (layer_a, layer_b):
        y = layer(x)
        assert y.shape == (2, m, 512)
        assert within_one_ulp(y, expect.to(torch.bfloat16))
        assert rel_l2(y, expect) <= 3 * REL_L2          # few outputs: single final-ulp flips weigh more


@pytest.mark.parametrize("m", [1, 4, 256])
def test_fused_mode_is_differentiable_in_the_activations(m):
    """The reference's forward is F.linear on a constant weight, so gradients flow to x (entropack/linear/linear.py:163-165).
    The fused mode's kernels are outside autograd; under it they run in a Function whose backward is grad @ W_dec. The
    input gradient must equal the decode_then_gemm layer's, which autograd derives from F.linear: the same bf16 product."""
    print("case fused backward, M =", m, flush=True)
    plain, _, _ = _c3_layer("decode_then_gemm", rows=512, cols=2048)
    fused, _, _ = _c3_layer("fused", rows=512, cols=2048)
    torch.manual_seed(21)
    x = torch.randn(m, 2048).to(torch.bfloat16).cuda()
    upstream = torch.randn(m, 512).to(torch.bfloat16).cuda()
    grads, outputs = [], []
    for layer in (plain, fused):
        probe = x.clone().requires_grad_(True)
        y = layer(probe)
        assert y.requires_grad
        y.backward(upstream)
        grads.append(probe.grad)
        outputs.append(y.detach())
    torch.cuda.synchronize()
    assert grads[1].shape == x.shape and grads[1].dtype == torch.bfloat16
    want = upstream.float() @ plain.dequantize("cuda").float()
    assert rel_l2(grads[0], want) <= REL_L2 and rel_l2(grads[1], want) <= REL_L2
    assert within_one_ulp(grads[1], want.to(torch.bfloat16))
    assert within_one_ulp(outputs[1], outputs[0])
    with torch.no_grad():                                            # and without autograd nothing is recorded
        assert not fused(x.clone().requires_grad_(True)).requires_grad


@pytest.mark.parametrize("rows,cols,bpp", [(512, 2048, 4.0), (96, 256, 3.0), (300, 1032, 8.0), (64, 4104, 2.0), (1024, 3072, 5.0)])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_fused_rows_never_materialise_the_weight_and_match(rows, cols, bpp, m):
    """One to four activation rows go through the multiply-on-the-fly decode kernel (every table kind that has one);
    the result must equal x @ bf16(W_dec).T + b to accumulation-order noise. Shapes cover row ends inside a group
    (cols / 8 not a multiple of 32), rows shorter and longer than a tile, and prob_bits 12."""
    from entropack_amd.backends import hip as hip_backend
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    print("case", rows, cols, bpp, m, flush=True)
    layer, _, bias = _c3_layer("fused", rows=rows, cols=cols, bpp=bpp)
    torch.manual_seed(13)
    x = torch.randn(m, cols).to(torch.bfloat16).cuda()
    decoded = layer.dequantize("cuda")
    expect = F.linear(x.float(), decoded.float(), bias.cuda().float())
    from entropack_amd.schemes.base import packed_buffers
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
    buffers = packed_buffers(layer.weight.buffers, LatticeBuffers)
    seen = []
    for kind in (None, hip_backend.TABLE_LDS_RANK, hip_backend.TABLE_LDS_WIDE, hip_backend.TABLE_LDS_SYM):
        hip_lane.FORCE_TABLE_KIND = kind
        try:
            # The kernel itself for every table kind; the layer's own choice (which may prefer decode + GEMM) once.
            y = hip_lane.linear_rows(buffers, shape=(rows, cols), x=x, bias=bias.cuda())
            y_layer = layer(x) if kind is None else y
        except hip_backend.HipError as error:
            if error.status != hip_backend.EUNSUPPORTED:
                raise
            continue
        finally:
            hip_lane.FORCE_TABLE_KIND = None
        torch.cuda.synchronize()
        hip_lane.check_errors(buffers)
        seen.append(kind)
        for got in (y, y_layer):
            assert got.shape == (m, rows) and got.dtype == torch.bfloat16
            assert within_one_ulp(got, expect.to(torch.bfloat16)), kind
            assert rel_l2(got, expect) <= 3 * REL_L2, kind                 # few outputs: single final-ulp flips weigh more
    assert None in seen and hip_backend.TABLE_LDS_RANK in seen


def test_fused_rows_direct_call_checks_and_f32_accuracy():
    """linear_rows itself: float32-level agreement of the accumulator path (bias-free, so the only rounding left is the
    final cast), batch-shaped activations, and the argument checks."""
    from entropack_amd.schemes.base import packed_buffers
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
    layer, _, _ = _c3_layer("fused", rows=384, cols=1024, bpp=4.0)
    container = layer.weight
    buffers = packed_buffers(container.buffers, LatticeBuffers)
    decoded = layer.dequantize("cuda").float()
    torch.manual_seed(14)
    x = torch.randn(2, 2, 1024).to(torch.bfloat16).cuda()
    y = hip_lane.linear_rows(buffers, shape=(384, 1024), x=x, bias=None)
    assert y.shape == (2, 2, 384)
    assert within_one_ulp(y, (x.float() @ decoded.T).to(torch.bfloat16))
    hip_lane.check_errors(buffers)
    with pytest.raises(ValueError):
        hip_lane.linear_rows(buffers, shape=(384, 1024), x=torch.randn(5, 1024).to(torch.bfloat16).cuda(), bias=None)
    with pytest.raises(ValueError):
        hip_lane.linear_rows(buffers, shape=(384, 1024), x=x.float(), bias=None)


@pytest.mark.parametrize("mode", ["decode_then_gemm", "fused"])
def test_int8_linear_forward_matches_its_definition(mode):
    layer, weight, bias = _c3_layer(mode, rows=1024, cols=1536, cls=ep.CompressedINT8Linear)
    torch.manual_seed(3)
    x = torch.randn(300, 1536).to(torch.bfloat16).cuda()
    y = layer(x)
    codes = layer.codes("cuda")
    assert codes.dtype == torch.int8 and codes.shape == (1024, 1536)
    flat = x.float().cpu()
    sa = (flat.abs().amax(dim=1) / torch.tensor(127.0)).clamp(min=torch.finfo(torch.float32).eps)
    qa = (flat / sa.unsqueeze(1)).round().clamp(-127, 127).cuda()
    sa = sa.cuda()
    expect = ((qa.double() @ codes.double().T).float() * sa.unsqueeze(1) * layer.weight_quant_scale.cuda().unsqueeze(0)
              + bias.cuda().float().unsqueeze(0)).to(torch.bfloat16)
    assert torch.equal(y, expect)
    # and the quantised layer still approximates the dense one
    assert rel_l2(y, F.linear(x.float(), weight.cuda().float(), bias.cuda().float())) < 0.15
    assert layer.weight_quant_scale.dtype == torch.float32
    layer.to(torch.float16)
    assert layer.weight_quant_scale.dtype == torch.float32        # Module.to must not cast the row scales


def _rotation(order):
    """Kronecker power of the 4 x 4 seed over sqrt(order), in float64 (entropack/linear/convrot.py:9-45 of the reference)."""
    seed = torch.tensor([[1.0, 1, 1, -1], [1, 1, -1, 1], [1, -1, 1, 1], [-1, 1, 1, 1]], dtype=torch.float64)
    matrix = seed
    while matrix.shape[0] < order:
        matrix = torch.kron(matrix, seed)
    return matrix / matrix.shape[0] ** 0.5


def _rotated_then_quantised(x, group):
    """Exact rotation (float64), rounded once to x's dtype, then the IEEE float32 row quantiser, all on the CPU."""
    flat = x.detach().cpu()
    rows, inner = flat.shape
    rotated = (flat.double().reshape(rows, inner // group, group) @ _rotation(group)).reshape(rows, inner).to(flat.dtype).float()
    scale = (rotated.abs().amax(dim=1) / torch.tensor(127.0)).clamp(min=torch.finfo(torch.float32).eps)
    return (rotated / scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8), scale


@pytest.mark.parametrize("group", [4, 16, 64, 256, 1024])
@pytest.mark.parametrize("rows,inner,dtype", [(300, 3072, torch.bfloat16), (5, 1024, torch.float32), (1, 2048, torch.float16), (33, 5120, torch.bfloat16)])
def test_rotate_quantize_rows_on_exactly_representable_sums(group, rows, inner, dtype):
    """Small integers: every partial sum is exact in float32 whatever the order, so the codes must be THE codes."""
    torch.manual_seed(group + rows)
    x = torch.randint(-8, 9, (rows, inner)).to(dtype).cuda()
    x[0, :] = 0
    codes, scale = kernels.rotate_quantize_rows(x, group)
    expect_codes, expect_scale = _rotated_then_quantised(x, group)
    assert torch.equal(scale.cpu(), expect_scale)
    assert torch.equal(codes.cpu(), expect_codes)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quantize_rows_of_two_byte_activations_is_the_divisions_answer_for_every_value(dtype):
    """The kernel for bfloat16 / float16 rows multiplies by 1 / scale and falls back to the division only where the product
    lies within 2^-14 of a half-integer. Rows whose maxima give scales that are no powers of two, filled with every value
    of the dtype up to the row's maximum (bfloat16: all of them; float16: every fourth), must come out as IEEE division,
    rint and clamp say, code for code."""
    bits = torch.arange(0, 0x7F80 if dtype == torch.bfloat16 else 0x7C00, 1 if dtype == torch.bfloat16 else 4, dtype=torch.int32)
    values = bits.to(torch.int16).view(dtype)
    tops = torch.tensor([0.37, 1.0, 3.1, 200.0, 1000.0, 4.4e-3, 77.0, 130.0, 513.0, 2.0e4], dtype=torch.float32).to(dtype)
    inner = 8192
    rows = []
    for top in tops:
        below = values[values.float() <= top.float()]
        signed = torch.cat([below, -below])
        pad = (-signed.numel()) % (inner - 1)
        signed = torch.cat([signed, signed.repeat(pad // signed.numel() + 1)[:pad]])
        block = signed.view(-1, inner - 1)
        rows.append(torch.cat([top.expand(block.shape[0], 1), block], dim=1))          # column 0 pins the row's maximum
    x = torch.cat(rows).contiguous().cuda()
    codes, scale = kernels.quantize_rows(x)
    flat = x.float().cpu()
    expect_scale = (flat.abs().amax(dim=1) / torch.tensor(127.0)).clamp(min=torch.finfo(torch.float32).eps)
    expect_codes = (flat / expect_scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)
    assert torch.equal(scale.cpu(), expect_scale)
    assert torch.equal(codes.cpu(), expect_codes)
    naive = (flat * (1.0 / expect_scale).unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)
    print("values a reciprocal multiply alone gets wrong:", int((naive != expect_codes).sum()), "of", naive.numel(), flush=True)


@pytest.mark.parametrize("group,rows,inner,dtype", [(256, 4096, 3072, torch.bfloat16), (64, 17, 3136, torch.bfloat16), (16, 9, 1008, torch.float16),
                                                    (4, 3, 4100, torch.float32), (256, 128, 28672, torch.bfloat16)])
def test_rotate_quantize_rows_on_gaussian_rows_with_outliers(group, rows, inner, dtype):
    """Float32 sums in butterfly order against the exact rotation: a value on a rounding boundary may move a code by one."""
    torch.manual_seed(group)
    x = torch.randn(rows, inner)
    x[:, 5] *= 40.0
    x = x.to(dtype).cuda()
    codes, scale = kernels.rotate_quantize_rows(x, group)
    expect_codes, expect_scale = _rotated_then_quantised(x, group)
    assert torch.allclose(scale.cpu(), expect_scale, rtol=2.0 ** -7 if dtype != torch.float32 else 1e-6, atol=0)
    same_scale = scale.cpu() == expect_scale
    assert same_scale.float().mean() >= 0.98
    delta = (codes.cpu().int() - expect_codes.int()).abs()[same_scale]
    assert int(delta.max()) <= 1
    assert float((delta != 0).float().mean()) <= 1e-3
    # the rotation spread the outlier channel: no code row is dominated by one entry any more
    plain_codes, _ = kernels.quantize_rows(x)
    assert float(codes.float().abs().mean()) > (2.0 if group >= 64 else 1.1) * float(plain_codes.float().abs().mean())


@pytest.mark.parametrize("mode", ["decode_then_gemm", "fused"])
def test_int8_linear_with_rotation_matches_its_definition(mode):
    """use_convrot: y = int8 product of the rotated-and-quantised activations with the codes of the rotated weight,
    exact in float32; and against the dense layer it is closer than the unrotated W8A8 layer when x has outlier channels."""
    torch.manual_seed(2)
    rows, cols = 768, 1536
    dense = torch.nn.Linear(cols, rows, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(rows, cols) * 0.02).to(torch.bfloat16))
    dense.bias.data.copy_((torch.randn(rows) * 0.01).to(torch.bfloat16))
    turned = ep.CompressedINT8Linear.from_linear(dense, forward_mode=mode, use_convrot=True).cuda()
    plain = ep.CompressedINT8Linear.from_linear(dense, forward_mode=mode).cuda()
    assert turned._convrot_group == 256
    x = torch.randn(300, cols)
    x[:, 11] *= 50.0
    x[:, 700] *= 30.0
    x = x.to(torch.bfloat16).cuda()
    y = turned(x)
    qa, sa = kernels.rotate_quantize_rows(x, 256)
    codes = turned.codes("cuda")
    expect = ((qa.double() @ codes.double().T).float() * sa.unsqueeze(1) * turned.weight_quant_scale.cuda().unsqueeze(0)
              + dense.bias.data.cuda().float().unsqueeze(0)).to(torch.bfloat16)
    assert torch.equal(y, expect)
    exact = F.linear(x.float(), dense.weight.data.cuda().float(), dense.bias.data.cuda().float())
    assert rel_l2(y, exact) < 0.5 * rel_l2(plain(x), exact)
    assert rel_l2(y, exact) < 0.03
    # the input gradient goes through the dequantised weight in the original basis
    probe = x[:4].clone().requires_grad_(True)
    turned(probe).float().sum().backward()
    assert rel_l2(probe.grad.float(), dense.weight.data.cuda().float().sum(dim=0).expand(4, cols)) < 0.05


def test_state_dict_round_trip_through_torch_save():
    """Usage/Linear-layers doc flow: save state_dict -> fresh layers -> torch.load(weights_only=True) -> same outputs."""
    layer, _, _ = _c3_layer("decode_then_gemm", rows=256, cols=512)
    model = torch.nn.Sequential(layer)
    state = model.state_dict()
    assert sorted(state) == ["0.bias", "0.weight.entropack_quant_state"]
    assert state["0.weight.entropack_quant_state"].dtype == torch.uint8 and state["0.weight.entropack_quant_state"].ndim == 1
    buffer = io.BytesIO()
    torch.save(state, buffer)
    buffer.seek(0)
    loaded = torch.load(buffer, weights_only=True)
    fresh = torch.nn.Sequential(ep.CompressedLinear(512, 256, config=ep.EntroPackLossyConfig(target_bpp=4.0), device="cuda"))
    result = fresh.load_state_dict(loaded)
    assert not result.missing_keys and not result.unexpected_keys
    x = torch.randn(8, 512, device="cuda").to(torch.bfloat16)
    assert torch.equal(fresh(x), model(x))
    assert fresh[0].weight.device.type == "cuda"
    empty = ep.CompressedLinear(512, 256, device="cuda")
    with pytest.raises(RuntimeError, match="nothing to decode"):
        empty(x)
    wrong = ep.CompressedLinear(256, 512, device="cuda")
    with pytest.raises(RuntimeError):
        torch.nn.Sequential(wrong).load_state_dict(loaded)
