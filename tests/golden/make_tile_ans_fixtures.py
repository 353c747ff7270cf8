"""Write the lossless (`tile_ans`) golden fixtures under tests/golden/tile_ans/ by running the upstream reference's
CPU (eager) lane.

Runs only in the build container, where the read-only reference checkout is mounted at /root/reference; nothing here
is needed (or present) on a GPU box. The reference ships no test vectors, and the conventions a decoder must share
with its encoder (word order inside a renormalisation step, tail group first, stream order, raw-lane packing, the
4096 -> 0 frequency escape, the precision and lane-mode choice) are pinned by nothing but its own output. Each fixture
records one small tensor: its raw bits, the config, the six container buffers the reference encoder wrote, the packed
`entropack_quant_state` blob, and the bits of what the reference's `decompress` returns (always the input: the codec
is lossless, which the script asserts).

Usage:  PYTHONDONTWRITEBYTECODE=1 python tests/golden/make_tile_ans_fixtures.py
"""
import os
import sys

import numpy as np
import torch

REFERENCE = "/root/reference"
OUT_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tile_ans")

_BITS = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def raw_bits(tensor: torch.Tensor) -> np.ndarray:
    tensor = tensor.detach().cpu().contiguous()
    if tensor.dtype == torch.bool:
        return tensor.numpy().astype(np.uint8)
    return tensor.view(_BITS[tensor.element_size()]).numpy().copy()


def cases():
    def gauss(seed, shape, sigma, dtype):
        torch.manual_seed(seed)
        return (torch.randn(*shape) * sigma).to(dtype)

    torch.manual_seed(40)
    yield "bf16_300x200_auto", gauss(41, (300, 200), 0.02, torch.bfloat16), {}
    yield "bf16_7x33_tile100", gauss(42, (7, 33), 0.02, torch.bfloat16), dict(tile_elements=100)
    yield "bf16_64x128_pb9", gauss(43, (64, 128), 0.02, torch.bfloat16), dict(probability_bits=9)
    yield "bf16_5x40_tile32", gauss(44, (5, 40), 1.0, torch.bfloat16), dict(tile_elements=32)
    yield "f16_64x96_auto", gauss(45, (64, 96), 0.02, torch.float16), {}
    yield "f32_40x72_auto", gauss(46, (40, 72), 0.02, torch.float32), {}
    yield "f32_3x5x7_tile64_pb12", gauss(47, (3, 5, 7), 3.0, torch.float32), dict(tile_elements=64, probability_bits=12)
    yield "int8_128x100_auto", (torch.randn(128, 100) * 30).round().clamp(-127, 127).to(torch.int8), {}
    yield "uint8_const_50x40_pb12", torch.full((50, 40), 7, dtype=torch.uint8), dict(probability_bits=12)
    yield "int64_10x10_auto", torch.randint(-50, 50, (10, 10), dtype=torch.int64), {}
    yield "bool_33x7_auto", torch.rand(33, 7) < 0.2, {}
    yield "int16_noise_60x50_auto", torch.randint(-32768, 32767, (60, 50), dtype=torch.int16), {}            # every lane raw
    yield "bf16_200x64_allcoded", gauss(48, (200, 64), 0.02, torch.bfloat16), dict(raw_lane_threshold=8.0)   # both lanes coded
    yield "f8e4m3_96x64_auto", gauss(49, (96, 64), 0.5, torch.float32).to(torch.float8_e4m3fn), {}
    yield "bf16_1x1_auto", gauss(50, (1, 1), 0.02, torch.bfloat16), {}
    yield "bf16_33x37_tile400", gauss(51, (33, 37), 0.02, torch.bfloat16), dict(tile_elements=400)           # coded, 21-element last tile
    yield "int16_steps_70x45_tile512_pb10", torch.randint(-300, 300, (70, 45), dtype=torch.int16) * 16, dict(tile_elements=512, probability_bits=10)
    yield "f32_50x60_tile1000_pb11", gauss(52, (50, 60), 0.02, torch.float32), dict(tile_elements=1000, probability_bits=11)
    yield "bf16_96x96_pb12", gauss(53, (96, 96), 0.02, torch.bfloat16), dict(probability_bits=12)


def main() -> int:
    sys.dont_write_bytecode = True
    sys.path.insert(0, REFERENCE)
    import entropack as reference          # the upstream package, CPU lane only (no CUDA here)

    os.makedirs(OUT_DIR, exist_ok=True)
    names = []
    for name, tensor, options in cases():
        config = reference.TileANSConfig(execution_backend="eager", **options)
        container = reference.compress(tensor, config)
        if container.compress_method != "tile_ans":
            raise SystemExit(f"{name}: reference fell back to {container.compress_method}")
        restored = reference.decompress(container, reference.TileANSConfig(execution_backend="eager"))
        if restored.dtype != tensor.dtype or tuple(restored.shape) != tuple(tensor.shape) or not np.array_equal(raw_bits(restored), raw_bits(tensor)):
            raise SystemExit(f"{name}: the reference's own round trip is not lossless")
        record = {
            "dtype": np.array(str(tensor.dtype).removeprefix("torch.")),
            "shape": np.array(tensor.shape, dtype=np.int64),
            "options_keys": np.array(sorted(options)),
            "options_values": np.array([float(options[k]) for k in sorted(options)], dtype=np.float64),
            "weight_bits": raw_bits(tensor),
            "quant_state": container.entropack_quant_state.detach().cpu().numpy().copy(),
        }
        for key, value in container.buffers.items():
            record["buf_" + key] = raw_bits(value) if value.dtype != torch.uint8 else value.cpu().numpy().copy()
        np.savez_compressed(os.path.join(OUT_DIR, name + ".npz"), **record)
        modes = container.buffers["lane_modes"].tolist()
        layout = container.buffers["layout"].tolist()
        print(f"{name}: layout {layout} lane_modes {modes} words {container.buffers['payload'].numel()}")
        names.append(name)
    with open(os.path.join(OUT_DIR, "INDEX.txt"), "w") as handle:
        handle.write("\n".join(names) + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
