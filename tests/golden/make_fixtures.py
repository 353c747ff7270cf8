"""Write the golden fixtures under tests/golden/ by running the upstream reference's CPU (eager) lane.

Runs only in the build container, where the read-only reference checkout is mounted at /root/reference;
nothing here is needed (or present) on a GPU box. The reference ships no test vectors of its own, and the
joint encoder/decoder conventions of its bitstream (lane<->word order inside a renormalisation step, field
order, tail-group-first schedule, Hamilton tie-breaking) are pinned by nothing but its own output, so each
fixture records, for one small tensor:

  * the input weight (raw bits), the config, the seven container buffers the reference encoder wrote,
  * the packed ``entropack_quant_state`` blob,
  * the symbol planes its entropy decoder returns (coset + 8 shifted fields),
  * the dense tensor ``decompress`` returns (raw bits), and ``actual_bpp``.

Usage:  PYTHONDONTWRITEBYTECODE=1 python tests/golden/make_fixtures.py [NAME_PREFIX]
"""
import os
import sys

import numpy as np
import torch

REFERENCE = "/root/reference"
OUT_DIR = os.path.dirname(os.path.abspath(__file__))

_BITS = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def raw_bits(tensor: torch.Tensor) -> np.ndarray:
    """Bit pattern of a tensor as a same-width integer numpy array (numpy has no bf16/fp8)."""
    tensor = tensor.detach().cpu().contiguous()
    if tensor.dtype == torch.bool:
        return tensor.numpy().astype(np.uint8)
    return tensor.view(_BITS[tensor.element_size()]).numpy().copy()


def cases():
    def gauss(seed, rows, cols, sigma, dtype=torch.bfloat16):
        torch.manual_seed(seed)
        return (torch.randn(rows, cols) * sigma).to(dtype)

    def outliers(seed, rows, cols, sigma, fraction=0.001, factor=20.0):
        torch.manual_seed(seed)
        weight = torch.randn(rows, cols) * sigma
        count = max(1, int(round(rows * cols * fraction)))
        index = torch.randperm(rows * cols)[:count]
        weight.view(-1)[index] *= factor
        return weight.to(torch.bfloat16)

    def int8_codes(seed, rows, cols):
        torch.manual_seed(seed)
        weight = torch.randn(rows, cols) * 0.02
        scale = weight.abs().amax(dim=1) / 127.0
        return (weight / scale.unsqueeze(1)).round().clamp(-127, 127).to(torch.int8)

    yield "c1_256x256_bf16_3p5", gauss(0, 256, 256, 0.02), dict(target_bpp=3.5)
    yield "ragged_66x200_bf16_4p0", gauss(11, 66, 200, 0.02), dict(target_bpp=4.0)
    yield "hi_96x512_bf16_8p0", gauss(12, 96, 512, 0.02), dict(target_bpp=8.0)
    yield "outlier_128x256_bf16_4p0", outliers(13, 128, 256, 0.02), dict(target_bpp=4.0)
    yield "codes_128x256_int8_4p0", int8_codes(14, 128, 256), dict(target_bpp=4.0)
    yield "zeros_16x64_bf16_4p0", torch.zeros(16, 64, dtype=torch.bfloat16), dict(target_bpp=4.0)
    yield "tiny_tiles_32x96_bf16_10p0", gauss(15, 32, 96, 0.02), dict(target_bpp=10.0, tile_elements=288)
    yield "wide_64x256_bf16_6p0", outliers(20, 64, 256, 0.02, 0.004, 60.0), dict(target_bpp=6.0)
    yield "huge_alpha_16x1024_bf16_7p0", outliers(21, 16, 1024, 0.02, 0.001, 5000.0), dict(target_bpp=7.0)
    yield "low_64x512_bf16_2p0", gauss(16, 64, 512, 0.02), dict(target_bpp=2.0)
    yield "f16_48x128_5p0", gauss(17, 48, 128, 0.5, torch.float16), dict(target_bpp=5.0)
    yield "f32_40x72_6p0_pb13", gauss(18, 40, 72, 1.5, torch.float32), dict(target_bpp=6.0, prob_bits=13)
    yield "pb9_64x128_bf16_1p5", gauss(19, 64, 128, 0.02), dict(target_bpp=1.5, prob_bits=9)
    # the optional per-row rate-distortion pass (row_rdo_iterations > 0)
    yield "rdo2_96x256_bf16_3p0", gauss(30, 96, 256, 0.02), dict(target_bpp=3.0, row_rdo_iterations=2)
    yield "rdo1_k3_64x512_bf16_4p0", outliers(31, 64, 512, 0.02, 0.002, 12.0), dict(target_bpp=4.0, row_rdo_iterations=1, row_rdo_candidates=3)
    yield "rdo3_k7_40x72_f32_5p0", gauss(32, 40, 72, 1.5, torch.float32), dict(target_bpp=5.0, row_rdo_iterations=3, row_rdo_candidates=7)
    yield "rdo2_rows_differ_128x128_bf16_2p5", (gauss(33, 128, 128, 0.02).float() * torch.logspace(-1, 1, 128).unsqueeze(1)).to(torch.bfloat16), dict(target_bpp=2.5, row_rdo_iterations=2)


def main() -> None:
    sys.dont_write_bytecode = True
    sys.path.insert(0, REFERENCE)
    import entropack as ep
    from entropack.schemes.lattice_rans import eager as ref_eager
    from entropack.schemes.lattice_rans import rans as ref_rans
    from entropack.schemes.lattice_rans.format import LatticeBuffers, decode_geometry, vector_tile_elements

    only = sys.argv[1] if len(sys.argv) > 1 else None        # a name prefix: write those fixtures only, keep the others
    names = []
    for name, weight, options in cases():
        if only is not None and not name.startswith(only):
            if os.path.exists(os.path.join(OUT_DIR, name + ".npz")):
                names.append(name)
            continue
        config = ep.EntroPackLossyConfig(execution_backend="eager", **options)
        compressed = ep.compress(weight, config)
        assert compressed.compress_method == "lattice_rans", compressed.header
        restored = ep.decompress(compressed, config)
        buffers = LatticeBuffers(**{key: compressed.buffers[key] for key in LatticeBuffers._fields})

        info = decode_geometry(buffers._asdict(), tuple(weight.shape))
        payload, offsets, states, meta, freq_tables, _scales = ref_eager._host_views(buffers)
        frequencies = ref_eager._stream_frequencies(freq_tables, meta)
        vectors = info["rows"] * (info["cols"] // 8)
        cosets, fields = ref_rans.decode_vector_stream(
            payload, offsets, states, frequencies, info["prob_bits"], vector_tile_elements(info["tile_elements"]), vectors,
        )
        record = {
            "weight_bits": raw_bits(weight),
            "restored_bits": raw_bits(restored),
            "dtype": np.array(str(weight.dtype).removeprefix("torch.")),
            "shape": np.array(weight.shape, dtype=np.int64),
            "options_keys": np.array(sorted(options)),
            "options_values": np.array([float(options[key]) for key in sorted(options)], dtype=np.float64),
            "actual_bpp": np.array(compressed.actual_bpp, dtype=np.float64),
            "quant_state": compressed.entropack_quant_state.detach().cpu().numpy().copy(),
            "cosets": cosets.astype(np.int8),
            "fields": fields.astype(np.int32),
        }
        for key in LatticeBuffers._fields:
            value = compressed.buffers[key].detach().cpu()
            record["buf_" + key] = raw_bits(value) if value.dtype in (torch.uint16, torch.uint32) else value.numpy().copy()
        np.savez_compressed(os.path.join(OUT_DIR, name + ".npz"), **record)
        names.append(name)
        print(f"{name}: shape={tuple(weight.shape)} bpp={compressed.actual_bpp:.4f} layout={compressed.buffers['layout'].tolist()} "
              f"tiles={states.shape[0]} words={payload.size} alphabets={meta[:, 3].tolist()}")
    with open(os.path.join(OUT_DIR, "INDEX.txt"), "w") as handle:
        handle.write("\n".join(names) + "\n")


if __name__ == "__main__":
    main()
