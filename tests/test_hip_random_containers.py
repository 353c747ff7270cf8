"""Differential run over randomly drawn containers: shapes, rates, table precisions, tile sizes, outliers and dtypes
are drawn from a fixed seed, encoded by the package's CPU encoder, decoded on the GPU and compared bit for bit with
the CPU oracle (lattice_rans) or with the oracle and the input (tile_ans)."""
import random

import numpy as np
import pytest
import torch

import entropack_amd as ep
from oracle import c_oracle

pytestmark = pytest.mark.gpu

_NAMES = {torch.bfloat16: "bfloat16", torch.float16: "float16", torch.float32: "float32"}


def _host(buffers):
    out = {}
    for key, value in buffers.items():
        if value.dtype in (torch.uint16, torch.uint32):
            signed = value.view(torch.int16 if value.dtype == torch.uint16 else torch.int32).numpy()
            out[key] = signed.view(np.uint16 if value.dtype == torch.uint16 else np.uint32)
        else:
            out[key] = value.numpy()
    return out


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_lattice_containers_match_the_oracle(seed):
    rng = random.Random(seed)
    c_oracle.load()
    for case in range(40):
        torch.manual_seed(rng.randrange(1 << 30))
        rows = rng.choice([1, 2, 3, 7, 16, 33, 100, 257, 512, 1000, 2048])
        cols = rng.choice([8, 16, 24, 40, 64, 100, 129, 256, 520, 1024, 3000, 4096, 7168])
        rows = min(rows, max(1, 3_000_000 // cols))
        weight = torch.randn(rows, cols) * rng.choice([1e-3, 0.02, 1.0, 30.0])
        if rng.random() < 0.3:
            picks = torch.randperm(rows * cols)[: max(1, rows * cols // 500)]
            weight.view(-1)[picks] *= rng.choice([8.0, 20.0, 60.0])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        options = dict(target_bpp=rng.choice([1.0, 1.7, 2.3, 3.0, 4.0, 5.0, 6.5, 8.0, 9.5]), execution_backend="eager")
        if rng.random() < 0.5:
            options["prob_bits"] = rng.choice([9, 10, 11, 12, 13, 14])
        if rng.random() < 0.5:
            options["tile_elements"] = rng.choice([288, 300, 1000, 4096, 9000, 16384, 40000])
        print("case", seed, case, rows, cols, dtype, options, flush=True)
        container = ep.compress(weight.to(dtype), ep.EntroPackLossyConfig(**options))
        assert container.compress_method == "lattice_rans"
        got = ep.decompress(container.to("cuda"), ep.EntroPackLossyConfig(execution_backend="hip")).cpu()
        expect = c_oracle.decode(_host(container.buffers), (rows, int(container.buffers["layout"][0])), _NAMES[dtype], threads=8)[:, :cols]
        if dtype == torch.float32:
            assert np.array_equal(got.view(torch.int32).numpy().view(np.uint32), expect.view(np.uint32))
        else:
            assert np.array_equal(got.view(torch.int16).numpy().view(np.uint16), expect)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_tile_ans_containers_are_lossless_and_match_the_oracle(seed):
    rng = random.Random(seed)
    c_oracle.load_tile_ans()
    dtypes = [torch.bfloat16, torch.float16, torch.float32, torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64, torch.bool,
              torch.float8_e4m3fn]
    for case in range(60):
        torch.manual_seed(rng.randrange(1 << 30))
        count = rng.choice([1, 5, 31, 32, 33, 255, 256, 257, 1000, 4096, 8191, 8192, 8193, 70000, 300001])
        dtype = rng.choice(dtypes)
        kind = rng.choice(["gauss", "small", "const", "noise"])
        if dtype == torch.bool:
            tensor = torch.rand(count) < rng.random()
        elif dtype.is_floating_point:
            tensor = {"gauss": torch.randn(count) * 0.05, "small": torch.randn(count) * 1e-3, "const": torch.full((count,), 1.5),
                      "noise": torch.rand(count) * 1e4}[kind].to(dtype)
        else:
            info = torch.iinfo(dtype)
            values = {"gauss": (torch.randn(count) * 20).round(), "small": torch.randint(0, 3, (count,)).float(), "const": torch.full((count,), 7.0),
                      "noise": torch.randint(max(info.min, -(1 << 30)), min(info.max, 1 << 30), (count,)).float()}[kind]
            tensor = values.clamp(info.min, info.max).to(dtype)
        options = dict(execution_backend="eager")
        if rng.random() < 0.6:
            options["tile_elements"] = rng.choice([32, 100, 256, 512, 1000, 4096, 8192, 20000])
        if rng.random() < 0.6:
            options["probability_bits"] = rng.choice([9, 10, 11, 12])
        if rng.random() < 0.3:
            options["raw_lane_threshold"] = rng.choice([0.0, 4.0, 8.0])
        print("case", seed, case, count, dtype, kind, options, flush=True)
        container = ep.compress(tensor, ep.TileANSConfig(**options))
        assert container.compress_method == "tile_ans"
        got = ep.decompress(container.to("cuda"), ep.TileANSConfig(execution_backend="hip")).cpu()
        as_bytes = (lambda t: t.to(torch.uint8) if t.dtype == torch.bool else t.contiguous().view(torch.uint8))
        want = as_bytes(tensor).numpy().reshape(-1)
        assert np.array_equal(as_bytes(got).numpy().reshape(-1), want)
        assert np.array_equal(c_oracle.tile_ans_decode(_host(container.buffers), tensor.element_size(), threads=4), want)
