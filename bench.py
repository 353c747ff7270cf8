"""Headline benchmark: lossy (lattice_rans) decode throughput on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload target|c2|c5a|c5b|c4|tile_ans|gemm|gemm_phases|fused_lds|encode|tile_ans_encode]

One "step" = one decode of the whole container (entropy decode + E8 reconstruction + BF16 store) from buffers
already resident in HBM. Prints ONE JSON line. `value` = algorithmic bytes (container bytes read + dense bytes
written) per second over the K timed steps; `roofline` prices the decode kernel's own duration (HIP events on the
launch stream) against 8 TB/s; `cpu_baseline` times the CPU oracle (C port of the reference's CPU decoder) on this
host's cores for the same container.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
#: Device copies of a container are rotated through until their compressed bytes add up to this much (the card's last-level
#: cache holds 256 MB).
ROTATING_INPUT_BYTES = 640 << 20

#: HBM bytes per decode launch from two rocprofv3 --pmc runs of this script (FETCH_SIZE, scaled by the factor a plain
#: 512 MiB copy in the same run calibrates it to, plus WRITE_SIZE): a measurement of the kernels as they were when the
#: named profile was taken. `csrc_sha16` names those sources; when the kernels have changed since, the figure is not
#: reported (`traffic` is null and `traffic_source` says why) instead of going stale silently.
MEASURED_TRAFFIC = {
    "target": {"bytes": 599_800_000, "profile": "profiles/decode_sym_target_4bpp_hbm_traffic.md", "csrc_sha16": "afaa16960905fbe8"},
    "tile_ans": {"bytes": 819_000_000, "profile": "profiles/decode_tile_ans_bf16_8192x28672_bench.md", "csrc_sha16": "f3f46eef72554c3a"},
}
#: The kernel sources a traffic figure depends on, per workload.
TRAFFIC_SOURCES = {
    "target": ("ep_common.hpp", "ep_store.hpp", "ep_decode_lds.hpp", "ep_decode_lds.hip", "ep_decode_sym.hip", "ep_plan.hip"),
    "tile_ans": ("ep_common.hpp", "ep_decode_lds.hpp", "ep_tile_ans.hip"),
}


def csrc_sha16(workload):
    import hashlib
    digest = hashlib.sha256()
    for name in TRAFFIC_SOURCES[workload]:
        with open(os.path.join(ROOT, "entropack_amd", "csrc", name), "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()[:16]


def measured_traffic(workload, forced_kind=None):
    """(`traffic`, `traffic_source`) of a roofline entry."""
    entry = MEASURED_TRAFFIC.get(workload)
    if entry is None or forced_kind is not None:
        return None, "not measured for this workload"
    now = csrc_sha16(workload)
    if now != entry["csrc_sha16"]:
        return None, f"{entry['profile']} holds {entry['bytes']} bytes for kernel sources {entry['csrc_sha16']}; they are {now} now"
    return entry["bytes"], f"{entry['profile']} (kernel sources {now})"


WORKLOADS = {
    # name: (rows, cols, sigma, seed, target_bpp, outliers)
    "target": (8192, 28672, 0.015, 4, 4.0, False),     # the shape/rate the 60 %-of-HBM target is quoted on
    "c2": (4096, 4096, 0.02, 1, 4.0, True),
    "c5a": (8192, 28672, 0.015, 4, 2.0, False),
    "c5b": (8192, 28672, 0.015, 4, 8.0, False),
    "small": (1024, 4096, 0.02, 7, 4.0, False),
}


def make_weight(rows, cols, sigma, seed, outliers):
    torch.manual_seed(seed)
    weight = torch.randn(rows, cols) * sigma
    if outliers:
        count = int(round(rows * cols * 0.001))
        index = torch.randperm(rows * cols)[:count]
        weight.view(-1)[index] *= 20.0
    return weight.to(torch.bfloat16)


def algorithmic_bytes(buffers, rows, cols_padded, out_itemsize):
    read = sum(t.numel() * t.element_size() for t in buffers.values())
    return read + rows * cols_padded * out_itemsize


def host_arrays(buffers):
    out = {}
    for key, value in buffers.items():
        value = value.detach().cpu()
        if value.dtype == torch.uint16:
            out[key] = value.view(torch.int16).numpy().view(np.uint16)
        elif value.dtype == torch.uint32:
            out[key] = value.view(torch.int32).numpy().view(np.uint32)
        else:
            out[key] = value.numpy()
    return out


def cpu_baseline(host, rows, cols_padded, alg_bytes, threads):
    """The C port of the reference's CPU decoder on this host, whole container, best of 2."""
    from oracle import c_oracle
    c_oracle.load()
    best = float("inf")
    for _ in range(2):
        start = time.perf_counter()
        dense = c_oracle.decode(host, (rows, cols_padded), "bfloat16", threads=threads)
        best = min(best, time.perf_counter() - start)
    return dense, {
        "value": round(alg_bytes / best / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"whole container ({rows}x{cols_padded}), C port of the reference CPU decoder, {threads} OpenMP threads, best of 2, {best:.3f} s",
    }


def python_loop_baseline(host, rows, cols_padded, alg_bytes, tiles_sampled=8):
    """The literal per-symbol Python loop (the shape of the reference's own eager lane) on a few tiles, 1 core."""
    from oracle import lattice_oracle as orc
    geo = orc.geometry(host["layout"], rows)
    tv, tiles = geo["tile_vectors"], geo["tiles"]
    take = min(tiles_sampled, tiles - 1) if tiles > 1 else 1
    freqs = orc.stream_frequencies(host["freq_tables"], host["stream_meta"].astype(np.int64))
    off = host["offsets"].astype(np.int64)
    start = time.perf_counter()
    orc.decode_symbols(host["payload"][off[0]:off[take]], off[:take + 1] - off[0], host["states"][:take], freqs,
                       geo["prob_bits"], tv, take * tv if take < tiles else geo["vectors"])
    seconds = time.perf_counter() - start
    whole = seconds * tiles / take
    return {"value": round(alg_bytes / whole / 1e9, 6), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{take} of {tiles} tiles through the per-symbol Python loop, {seconds:.2f} s, scaled linearly in tiles"}


MFMA_PEAK_BF16_TFLOPS = 2500.0


#: Seconds of untimed launches in front of every timed region. From idle the card's clock governor needs about 30 ms of
#: load before launch times settle (8192x28672 @ 4 bpp decode: launches 5..25 after idle take 142-165 us, from the 200th
#: on 130 us, steady for as long as the load lasts); measurements taken inside that ramp describe the governor.
SETTLE_SECONDS = 0.2


def settle(fn, seconds=None):
    """Keeps the device busy with `fn` for `seconds` (queue kept full, one synchronisation per 32 calls)."""
    seconds = SETTLE_SECONDS if seconds is None else seconds
    started = time.perf_counter()
    while time.perf_counter() - started < seconds:
        for _ in range(32):
            fn()
        torch.cuda.synchronize()


def _median_ms(fn, steps, warmup=5, from_idle=False):
    """Median duration of `fn` over `steps` calls bracketed one by one, with the clocks settled; `from_idle`: after half a
    second without work instead (the first few tens of milliseconds of load run at other clocks: a decode slower, a
    matrix-core product faster, than they do in a loop that lasts)."""
    if from_idle:
        torch.cuda.synchronize()
        time.sleep(0.5)
    else:
        settle(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for begin, end in events:
        begin.record()
        fn()
        end.record()
    torch.cuda.synchronize()
    times = sorted(begin.elapsed_time(end) for begin, end in events)
    return times[len(times) // 2]


def linear_section(ep, steps):
    """Benchmark configuration 3: W 3072x3072 @ 4 bpp + bias, X [4096, 3072] bf16, seed 2; whole forward (decode + GEMM)."""
    from torch.nn import functional as F
    torch.manual_seed(2)
    dense = torch.nn.Linear(3072, 3072, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(3072, 3072) * 0.02).to(torch.bfloat16))
    dense.bias.data.copy_((torch.randn(3072) * 0.01).to(torch.bfloat16))
    x = torch.randn(4096, 3072).to(torch.bfloat16).cuda()
    flops = 2.0 * 4096 * 3072 * 3072
    out = {"workload": "CompressedLinear 3072x3072 @ 4.0 bpp + bias, X [4096, 3072] bf16, seed 2", "flops": flops}
    from entropack_amd.linear import fused as fused_mode
    reference = None
    # `fused` multiplies with the mode's default (fused.TILED_PRODUCT = "auto": this library's kernel where it runs blocks of
    # 64 x 64, e.g. 256 rows of this layer, the vendor library's otherwise); `fused_own_gemm` = the mode made to multiply with
    # this library's tiled kernels whatever the shape ("own").
    # `fused_through_lds` = the one kernel in which the matrix cores multiply decoded tiles taken from LDS (the dense weight is
    # never written); selected by name only, because it is the slower one.
    variants = (("decode_then_gemm", "decode_then_gemm", "library"), ("fused", "fused", "auto"), ("fused_own_gemm", "fused", "own"),
                ("fused_through_lds", "fused_through_lds", "library"))
    for name, mode, product in variants:
        layer = ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0), forward_mode=mode).cuda()
        fused_mode.TILED_PRODUCT = product
        y = layer(x)
        if reference is None:
            weight = layer.dequantize("cuda")
            reference = F.linear(x.float(), weight.float(), layer.bias.float()).to(torch.bfloat16).double()
            decode_ms = _median_ms(lambda: layer.dequantize("cuda"), steps)
            out["decode_ms"] = round(decode_ms, 5)
        rel = ((y.double() - reference).norm() / reference.norm()).item()
        ms = _median_ms(lambda: layer(x), steps)
        out[name] = {"ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 2),
                     "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_BF16_TFLOPS, 5), "rel_l2_vs_f32_reference": rel}
    # Fewer activation rows than the configuration names, between the 128 of the streaming kernel and the 4096 above.
    out["fewer_rows"] = {}
    for rows in (256, 1024):
        part = x[:rows].contiguous()
        entry = {}
        for name, mode, product in variants:
            layer = ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0), forward_mode=mode).cuda()
            fused_mode.TILED_PRODUCT = product
            got = layer(part).double()
            entry[name] = {"ms": round(_median_ms(lambda: layer(part), steps), 5),
                           "rel_l2_vs_f32_reference": ((got - reference[:rows]).norm() / reference[:rows].norm()).item()}
        out["fewer_rows"][f"M={rows}"] = entry
    fused_mode.TILED_PRODUCT = "auto"
    # The same layer encoded with tiles a quarter and an eighth of the default size (`tile_elements`, a field of the
    # reference's config): a tile's chain of dependent steps, which is all a single layer's decode waits for, shortens
    # in proportion, for a per-tile header that costs 1-3 % more stored bits.
    out["smaller_tiles"] = {}
    for tile_elements in (4096, 2048):
        config = ep.EntroPackLossyConfig(target_bpp=4.0, tile_elements=tile_elements)
        layer = ep.CompressedLinear.from_linear(dense, config=config, forward_mode="decode_then_gemm").cuda()
        y = layer(x)
        own = F.linear(x.float(), layer.dequantize("cuda").float(), layer.bias.float()).to(torch.bfloat16).double()
        ms = _median_ms(lambda: layer(x), steps)
        out["smaller_tiles"][f"tile_elements={tile_elements}"] = {
            "stored_bits_per_weight": round(layer.compressed_bits, 3), "decode_ms": round(_median_ms(lambda: layer.dequantize("cuda"), steps), 5),
            "ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 2), "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_BF16_TFLOPS, 5),
            "rel_l2_vs_f32_reference": ((y.double() - own).norm() / own.norm()).item()}
        layer.forward_mode = "fused_through_lds"
        y = layer(x)
        ms = _median_ms(lambda: layer(x), steps)
        out["smaller_tiles"][f"tile_elements={tile_elements}"]["fused_through_lds"] = {
            "ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 2), "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_BF16_TFLOPS, 5),
            "rel_l2_vs_f32_reference": ((y.double() - own).norm() / own.norm()).item()}
    # The same layer with its weight stored losslessly (tile_ans, the scheme a layer takes when given no config).
    layer = ep.CompressedLinear.from_linear(dense).cuda()
    y = layer(x)
    exact = F.linear(x.float(), dense.weight.data.cuda().float(), dense.bias.data.cuda().float()).to(torch.bfloat16).double()
    ms = _median_ms(lambda: layer(x), steps)
    out["lossless_decode_then_gemm"] = {
        "ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 2), "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_BF16_TFLOPS, 5),
        "decode_ms": round(_median_ms(lambda: layer.dequantize("cuda"), steps), 5), "stored_bits_per_weight": round(layer.compressed_bits, 3),
        "rel_l2_vs_dense_layer": ((y.double() - exact).norm() / exact.norm()).item()}
    return out


MFMA_PEAK_INT8_TOPS = 5000.0


def int8_linear_section(ep, steps):
    """Configuration 3's layer as W8A8 (`CompressedINT8Linear`, int8 codes lattice-coded at 4 bpp, per-row activation
    quantiser, int8 matrix cores): whole forward in both modes, against the layer's own definition in float64."""
    from entropack_amd.linear import kernels
    torch.manual_seed(2)
    dense = torch.nn.Linear(3072, 3072, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(3072, 3072) * 0.02).to(torch.bfloat16))
    dense.bias.data.copy_((torch.randn(3072) * 0.01).to(torch.bfloat16))
    x = torch.randn(4096, 3072).to(torch.bfloat16).cuda()
    ops = 2.0 * 4096 * 3072 * 3072
    out = {"workload": "CompressedINT8Linear 3072x3072, codes @ 4.0 bpp, + bias, X [4096, 3072] bf16, seed 2", "ops": ops}
    for mode in ("decode_then_gemm", "fused", "fused_through_lds"):
        layer = ep.CompressedINT8Linear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0), forward_mode=mode).cuda()
        y = layer(x)
        codes, (qa, sa) = layer.codes("cuda"), kernels.quantize_rows(x)
        definition = ((qa.double() @ codes.double().T) * sa.double().unsqueeze(1) * layer.weight_quant_scale.cuda().double().unsqueeze(0)
                      + dense.bias.data.cuda().double())
        rounded = definition.float().to(torch.bfloat16).double()                  # the layer rounds its float32 result once
        rel = ((y.double() - rounded).norm() / rounded.norm()).item()
        dense_rel = ((y.double() - torch.nn.functional.linear(x.double(), dense.weight.data.cuda().double(), dense.bias.data.cuda().double())).norm()
                     / definition.norm()).item()
        ms = _median_ms(lambda: layer(x), steps)
        out[mode] = {"ms": round(ms, 5), "tops": round(ops / ms / 1e9, 2), "frac_of_int8_mfma_peak": round(ops / ms / 1e9 / MFMA_PEAK_INT8_TOPS, 5),
                     "rel_l2_vs_definition_in_bf16": rel, "rel_l2_vs_dense_layer": dense_rel}
    out["quantize_rows_ms"] = round(_median_ms(lambda: kernels.quantize_rows(x), steps), 5)
    out["int8_gemm_ms"] = round(_median_ms(lambda: kernels.int8_gemm(qa, codes, sa, layer.weight_quant_scale.cuda(), None, torch.bfloat16), steps), 5)

    # The same layer as a stack of 48 (own device buffers each), code containers decoded 16 at a time: three groups, so
    # with two arenas every pass decodes every layer. `beside` = on a second stream while the previous group multiplies,
    # `in_line` = on the layers' own stream between two groups (one arena).
    import copy
    layer.forward_mode = "decode_then_gemm"                # the stack is the layer in its default mode
    stack = [copy.deepcopy(layer).cuda() for _ in range(48)]

    def forward():
        y = None
        for member in stack:
            y = member(x)
        return y

    reference = forward()
    alone = _median_ms(forward, max(3, steps // 5), warmup=2) / len(stack)
    entry = {"layer_by_layer_ms_per_layer": round(alone, 5)}
    best = None
    for name, overlap in (("beside", True), ("in_line", False)):
        with ep.DecodeAhead(stack, group_size=16, overlap=overlap) as ahead:
            same = bool(torch.equal(forward(), reference))
            ahead_ms = _median_ms(forward, max(3, steps // 5), warmup=2) / len(stack)
            ahead.check_errors()
            entry[f"decode_ahead_group_16_{name}"] = {"ms_per_layer": round(ahead_ms, 5), "identical_to_layer_by_layer": same,
                                                      "dense_bytes_held": ahead.arena_bytes}
        best = ahead_ms if best is None else min(best, ahead_ms)
    entry["tops"] = round(ops / best / 1e9, 2)
    entry["frac_of_int8_mfma_peak"] = round(ops / best / 1e9 / MFMA_PEAK_INT8_TOPS, 5)
    out["stack_of_48"] = entry
    return out


def stack_linear_section(ep, steps, layers_total=48, distinct=4):
    """Config 3's layer repeated as a stack (M = 4096, 3072 x 3072 @ 4 bpp + bias): a model's forward, where the weights of
    `group` layers are decoded per pass, beside the previous group's products or between two groups (DecodeAhead). Per-layer
    time over the whole stack; every pass decodes every layer (the stack has more than two groups)."""
    import copy
    torch.manual_seed(2)
    protos = []
    for _ in range(distinct):
        dense = torch.nn.Linear(3072, 3072, dtype=torch.bfloat16)
        dense.weight.data.copy_((torch.randn(3072, 3072) * 0.02).to(torch.bfloat16))
        dense.bias.data.copy_((torch.randn(3072) * 0.01).to(torch.bfloat16))
        protos.append(ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0)))
    layers = [copy.deepcopy(protos[index % distinct]).cuda() for index in range(layers_total)]      # own device buffers each
    x = torch.randn(4096, 3072).to(torch.bfloat16).cuda()
    flops = 2.0 * 4096 * 3072 * 3072

    def forward():
        out = None
        for layer in layers:
            out = layer(x)
        return out

    def priced(ms_stack, ms_stack_from_idle=None):
        per_layer = ms_stack / layers_total
        entry = {"ms_per_layer": round(per_layer, 5), "tflops": round(flops / per_layer / 1e9, 2),
                 "frac_of_mfma_peak": round(flops / per_layer / 1e9 / MFMA_PEAK_BF16_TFLOPS, 5)}
        if ms_stack_from_idle is not None:
            entry["ms_per_layer_from_idle"] = round(ms_stack_from_idle / layers_total, 5)
        return entry

    def both(fn):
        count = max(3, steps // 5)
        return priced(_median_ms(fn, count, warmup=2), _median_ms(fn, count, warmup=2, from_idle=True))

    out = {"workload": f"{layers_total} x CompressedLinear 3072x3072 @ 4.0 bpp + bias, X [4096, 3072] bf16, decode_then_gemm"}
    reference = forward()
    out["clocks"] = (f"ms_per_layer: after {SETTLE_SECONDS} s of the same forward passes (the card then runs at its 1400 W limit); "
                     "ms_per_layer_from_idle: the first passes after half a second without work")
    out["layer_by_layer"] = both(forward)
    weights = [layer.dequantize("cuda") for layer in layers[:distinct]]
    out["dense_gemm_only"] = both(lambda: [torch.nn.functional.linear(x, weights[i % distinct], layers[i].bias) for i in range(layers_total)])
    from entropack_amd.linear import fused as fused_mode
    from entropack_amd.linear import kernels
    out["dense_own_gemm_only"] = both(lambda: [kernels.gemm_bf16(x, weights[i % distinct], layers[i].bias) for i in range(layers_total)])
    del weights
    # `beside`: groups decode on a second stream while the previous group multiplies (two arenas); `in_line`: on the
    # layers' own stream between two groups (one arena).
    for group, overlap in ((8, True), (16, True), (16, False)):
        if layers_total // group < 3:
            continue
        with ep.DecodeAhead(layers, group_size=group, overlap=overlap) as ahead:
            same = bool(torch.equal(forward(), reference))
            entry = both(forward)
            entry["identical_to_layer_by_layer"] = same
            entry["dense_bytes_held"] = ahead.arena_bytes
            ahead.check_errors()
        out[f"decode_ahead_group_{group}" + ("" if overlap else "_in_line")] = entry
    # The same stack multiplied by this library's tiled kernel (fused mode, TILED_PRODUCT = "own") instead of the vendor's.
    for layer in layers:
        layer.forward_mode = "fused"
    fused_mode.TILED_PRODUCT = "own"
    try:
        own_reference = forward()
        rel = ((own_reference.double() - reference.double()).norm() / reference.double().norm()).item()
        with ep.DecodeAhead(layers, group_size=16, overlap=False) as ahead:
            same = bool(torch.equal(forward(), own_reference))
            entry = both(forward)
            entry["identical_to_layer_by_layer"] = same
            entry["rel_l2_vs_library_product"] = rel
            ahead.check_errors()
        out["decode_ahead_group_16_in_line_own_gemm"] = entry
    finally:
        fused_mode.TILED_PRODUCT = "auto"
        for layer in layers:
            layer.forward_mode = "decode_then_gemm"
    return out


def small_m_section(ep, on_gpu, rows, cols, bpp, steps):
    """Benchmark configuration 5, linear part: X [M, cols] bf16 N(0, 1), M in {1, 16, 128}, on the container just decoded.

    The weight stream bounds this regime, so each mode is priced in GB/s on the bytes it has to move: fused = the
    compressed container + x + y; decode_then_gemm adds one write and one read of the dense weight.
    """
    from torch.nn import functional as F
    compressed_bytes = sum(t.numel() * t.element_size() for t in on_gpu.buffers.values())
    dense_bytes = rows * cols * 2
    out = {"workload": f"CompressedLinear {rows}x{cols} @ {bpp} bpp, X [M, {cols}] bf16 N(0,1), seed 4"}
    layers = {}
    modes = ("decode_then_gemm", "fused") + (("fused_through_lds",) if bpp <= 7.0 else ())      # prob_bits 12 has no two-level tables
    for mode in modes:
        layer = ep.CompressedLinear(cols, rows, bias=False, device="cuda", dtype=torch.bfloat16, forward_mode=mode)
        layer.weight = torch.nn.Parameter(on_gpu, requires_grad=False)
        layers[mode] = layer
    weight = layers["fused"].dequantize("cuda").double()
    torch.manual_seed(4)
    for m in (1, 4, 16, 128):
        x = torch.randn(m, cols).to(torch.bfloat16).cuda()
        reference = F.linear(x.double(), weight).to(torch.bfloat16).double()      # float64 accumulation, rounded once
        entry = {}
        for mode, layer in layers.items():
            y = layer(x)
            rel = ((y.double() - reference).norm() / reference.norm()).item()
            ms = _median_ms(lambda: layer(x), max(5, steps // 2), warmup=2)
            moved = compressed_bytes + 2 * m * cols + 2 * m * rows
            if mode == "decode_then_gemm" or (mode == "fused" and m > 4):
                moved += 2 * dense_bytes
            entry[mode] = {"ms": round(ms, 5), "GBps_on_bytes_moved": round(moved / ms / 1e6, 1),
                           "tflops": round(2.0 * m * rows * cols / ms / 1e9, 3), "rel_l2_vs_f64_reference": rel}
        out[f"M={m}"] = entry
    del weight
    return out


STACK_SHAPES = ((11520, 3840), (3840, 3840), (10240, 3840), (3840, 10240))      # qkv, out, ffn-up, ffn-down as [out, in]
STACK_RATES = (2.3, 4.0, 5.0, 6.0, 8.0)


def stack_workload(args, ep):
    """Benchmark configuration 4: `--stack-blocks` blocks x 4 layers, N(0, 0.02) seed 3, rates round-robin; one pass decodes all."""
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    torch.manual_seed(3)
    containers, params, alg_bytes, kinds, check = [], 0, 0, {}, []
    started = time.perf_counter()
    for index in range(args.stack_blocks * 4):
        rows, cols = STACK_SHAPES[index % 4]
        rate = STACK_RATES[index % 5]
        weight = (torch.randn(rows, cols) * 0.02).to(torch.bfloat16)
        container = ep.compress(weight, ep.EntroPackLossyConfig(target_bpp=rate, execution_backend="eager"))
        params += rows * cols
        layer_bytes = algorithmic_bytes(container.buffers, rows, int(container.buffers["layout"][0]), 2)
        alg_bytes += layer_bytes
        if index < 5 and not args.no_cpu:
            check.append((index, host_arrays(container.buffers), rows, int(container.buffers["layout"][0]), layer_bytes))
        containers.append(container.to(device))
        if index % 10 == 9:
            print(f"encoded {index + 1} layers, {time.perf_counter() - started:.0f} s", file=sys.stderr, flush=True)
    encode_seconds = time.perf_counter() - started

    config = ep.EntroPackLossyConfig(execution_backend="hip")
    torch.cuda.synchronize()
    plan_started = time.perf_counter()
    batch = ep.BatchDecompressor(containers, config)          # per-container table builds + the batch plan: the cold start
    torch.cuda.synchronize()
    plan_seconds = time.perf_counter() - plan_started
    arena = torch.empty(batch.arena_bytes, dtype=torch.uint8, device=device)
    for container in containers:
        lattice = LatticeBuffers(**{key: container.buffers[key] for key in LatticeBuffers._fields})
        kind = hip_lane.plan_of(lattice).table_kind
        kinds[kind] = kinds.get(kind, 0) + 1

    def timed(fn, steps, warmup):
        settle(fn)
        for _ in range(max(warmup, 1)):
            out = fn()
        torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        wall = time.perf_counter()
        first.record()
        for _ in range(steps):
            out = fn()
        last.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - wall) / steps
        return out, wall, first.elapsed_time(last) / steps

    steps = min(args.steps, 20)
    dense, wall, device_ms = timed(lambda: batch(arena), steps, args.warmup)
    batch.check_errors()
    _, layer_wall, layer_ms = timed(lambda: [ep.decompress(c, config) for c in containers], max(2, steps // 4), 1)

    result = {
        "metric": "lossy decode GB/s (+% HBM roofline); CompressedLinear TFLOPS @ M=4096, 4 bpp",
        "value": round(alg_bytes / wall / 1e9, 3), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u32",
        "data": "synthetic",
        "config": {
            "workload": f"lattice_rans decode to bf16 of a DiT-like stack in one pass: {args.stack_blocks} blocks x "
                        f"{{11520x3840, 3840x3840, 10240x3840, 3840x10240}} N(0,0.02) seed 3, rates {list(STACK_RATES)} round-robin",
            "layers": len(containers), "params": params, "algorithmic_bytes": alg_bytes, "table_kinds": kinds,
            "params_per_s": round(params / wall, 1), "encode_seconds_cpu": round(encode_seconds, 1),
            "plan_build_ms_once": round(plan_seconds * 1e3, 2),
            "layer_by_layer": {"ms_per_pass": round(layer_wall * 1e3, 4), "device_ms": round(layer_ms, 4),
                               "GBps": round(alg_bytes / layer_wall / 1e9, 3)},
        },
        "roofline": {
            "bound": "hbm", "achieved": round(alg_bytes / (device_ms * 1e-3) / 1e9, 3), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(alg_bytes / (device_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5), "traffic": None,
            "kernel_ms_avg": round(device_ms, 5),
        },
    }
    if check:
        from oracle import c_oracle
        c_oracle.load()
        exact = True
        cpu_seconds, cpu_bytes = 0.0, 0
        for index, host, rows, cols_padded, layer_bytes in check:
            begin = time.perf_counter()
            expect = c_oracle.decode(host, (rows, cols_padded), "bfloat16", threads=min(16, os.cpu_count() or 1))
            cpu_seconds += time.perf_counter() - begin
            cpu_bytes += layer_bytes
            got = dense[index].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
            exact = exact and bool(np.array_equal(got, expect[:, :got.shape[1]]))
        result["config"]["bit_exact_vs_oracle_first_5_layers"] = exact
        result["cpu_baseline"] = {
            "value": round(cpu_bytes / cpu_seconds / 1e9, 4), "unit": "GB/s", "cores": min(16, os.cpu_count() or 1), "kind": "port",
            "sample": f"the first 5 layers (one per rate), C port of the reference CPU decoder, OpenMP, {cpu_seconds:.2f} s"}
    print(json.dumps(result))
    return 0 if parity_holds(result) else 1


def decode_case(ep, name, steps, warmup, check, small_m=False):
    """One decode-only configuration (a row of `decode_configs`): encode on the host, decode on the device, time the
    launches with HIP events, compare the result with the C oracle bit for bit."""
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers
    rows, cols, sigma, seed, bpp, outliers = WORKLOADS[name]
    container = ep.compress(make_weight(rows, cols, sigma, seed, outliers), ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager"))
    on_gpu = container.to("cuda")
    lattice = LatticeBuffers(**{key: on_gpu.buffers[key] for key in LatticeBuffers._fields})
    cols_padded = int(container.buffers["layout"][0])
    alg_bytes = algorithmic_bytes(container.buffers, rows, cols_padded, 2)

    def step():
        return hip_lane.decode(lattice, shape=(rows, cols), dtype=torch.bfloat16)

    dense = step()
    settle(step)
    for _ in range(max(warmup, 1)):
        dense = step()
    torch.cuda.synchronize()
    hip_lane.check_errors(lattice)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first.record()
    for _ in range(steps):
        dense = step()
    last.record()
    torch.cuda.synchronize()
    avg_ms = first.elapsed_time(last) / steps
    # The same launches rotating through device copies of the container (see main()).
    copies = max(2, -(-ROTATING_INPUT_BYTES // max(1, alg_bytes - 2 * rows * cols_padded)))
    rotating = [lattice] + [LatticeBuffers(**{key: one.buffers[key] for key in LatticeBuffers._fields})
                            for one in (container.to("cuda") for _ in range(min(copies, 48) - 1))]
    turn = [0]

    def rotating_step():
        turn[0] = (turn[0] + 1) % len(rotating)
        return hip_lane.decode(rotating[turn[0]], shape=(rows, cols), dtype=torch.bfloat16)

    for _ in rotating:
        rotating_step()
    settle(rotating_step)
    torch.cuda.synchronize()
    first.record()
    for _ in range(steps):
        rotating_step()
    last.record()
    torch.cuda.synchronize()
    rotating_ms = first.elapsed_time(last) / steps
    del rotating
    entry = {
        "workload": f"{rows}x{cols} N(0,{sigma}) seed {seed}{' +0.1% x20 outliers' if outliers else ''} @ {bpp} bpp -> bf16",
        "tiles": int(lattice.states.shape[0]), "prob_bits": int(container.buffers["layout"][1]),
        "table_kind": hip_lane.launch_table_kind(lattice, shape=(rows, cols), dtype=torch.bfloat16),
        # kernel_ms_avg / frac_of_hbm_peak: every launch reads its container from memory (device copies in turn), as for
        # the headline; *_same_container: one container over and over, its compressed bytes in the last-level cache.
        "algorithmic_bytes": alg_bytes, "kernel_ms_avg": round(rotating_ms, 5), "GBps": round(alg_bytes / rotating_ms / 1e6, 1),
        "frac_of_hbm_peak": round(alg_bytes / rotating_ms / 1e6 / HBM_PEAK_GBPS, 5), "params_per_s": round(rows * cols / (rotating_ms * 1e-3), 1),
        "kernel_ms_avg_same_container": round(avg_ms, 5),
        "frac_of_hbm_peak_same_container": round(alg_bytes / avg_ms / 1e6 / HBM_PEAK_GBPS, 5),
    }
    if check:
        from oracle import c_oracle
        c_oracle.load()
        expect = c_oracle.decode(host_arrays(container.buffers), (rows, cols_padded), "bfloat16", threads=min(16, os.cpu_count() or 1))
        entry["bit_exact_vs_oracle"] = bool(np.array_equal(dense.view(torch.int16).cpu().numpy().view(np.uint16), expect[:, :cols]))
        del expect
    del dense
    if small_m:
        entry["linear_small_m"] = small_m_section(ep, on_gpu, rows, cols, bpp, steps)
    return entry


def stack_case(ep, steps, check):
    """Configuration 4 inside the default run: 120 layers, rates round-robin, one batched pass. The 20 distinct
    (shape, rate) pairs are encoded once from one N(0, 0.02) weight per shape and every pair is placed on the device six
    times, as six layers with buffers and plans of their own: the decode work of the configuration without 120 encodes
    (`--workload c4` encodes 120 different weights)."""
    torch.manual_seed(3)
    weights = [(torch.randn(rows, cols) * 0.02).to(torch.bfloat16) for rows, cols in STACK_SHAPES]
    distinct = {}
    for index in range(20):
        distinct[index % 4, index % 5] = ep.compress(weights[index % 4], ep.EntroPackLossyConfig(target_bpp=STACK_RATES[index % 5],
                                                                                                 execution_backend="eager"))
    del weights
    keys = [(index % 4, index % 5) for index in range(120)]
    containers = [distinct[key].to("cuda") for key in keys]
    params = sum(STACK_SHAPES[key[0]][0] * STACK_SHAPES[key[0]][1] for key in keys)
    alg_bytes = sum(algorithmic_bytes(distinct[key].buffers, STACK_SHAPES[key[0]][0], int(distinct[key].buffers["layout"][0]), 2) for key in keys)
    config = ep.EntroPackLossyConfig(execution_backend="hip")
    torch.cuda.synchronize()
    plan_started = time.perf_counter()
    batch = ep.BatchDecompressor(containers, config)
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - plan_started) * 1e3
    arena = torch.empty(batch.arena_bytes, dtype=torch.uint8, device="cuda")
    dense = batch(arena)
    torch.cuda.synchronize()
    batch.check_errors()
    ms = _median_ms(lambda: batch(arena), max(5, steps // 5), warmup=2)
    entry = {
        "workload": "120 layers {11520x3840, 3840x3840, 10240x3840, 3840x10240} N(0,0.02) seed 3, rates [2.3, 4, 5, 6, 8] round-robin, "
                    "one batched pass (20 distinct containers, six device copies each)",
        "layers": len(containers), "params": params, "algorithmic_bytes": alg_bytes, "ms_per_pass": round(ms, 4),
        "GBps": round(alg_bytes / ms / 1e6, 1), "frac_of_hbm_peak": round(alg_bytes / ms / 1e6 / HBM_PEAK_GBPS, 5),
        "params_per_s": round(params / (ms * 1e-3), 1), "plan_build_ms_once": round(plan_ms, 2),
    }
    if check:
        from oracle import c_oracle
        c_oracle.load()
        exact = True
        for index in range(20):
            key = keys[index]
            rows, cols = STACK_SHAPES[key[0]]
            expect = c_oracle.decode(host_arrays(distinct[key].buffers), (rows, int(distinct[key].buffers["layout"][0])), "bfloat16",
                                     threads=min(16, os.cpu_count() or 1))
            got = dense[index].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
            exact = exact and bool(np.array_equal(got, expect[:, :cols]))
        for index in range(20, 120):                                  # the other copies against the checked ones
            exact = exact and bool(torch.equal(dense[index].view(torch.int16), dense[index % 20].view(torch.int16)))
        entry["bit_exact_vs_oracle"] = exact
    return entry


def gemm_workload(args, ep):
    """The tiled bf16 products on their own: this library's kernel and the vendor library's on the config-3 layer shape
    (N = K = 3072) at 256, 1024 and 4096 activation rows, once with one weight used over and over (operands resident in
    the caches) and once rotating through enough different weights that each one comes from memory, as a weight fresh from
    the decoder does; then the same product at M = 4096 against K, which separates the per-launch cost from the cost of
    a K step. Device times: 200 launches back to back between one pair of events, after the clocks have settled."""
    from torch.nn import functional as F
    from entropack_amd.linear import kernels
    torch.manual_seed(0)

    def timed(fn, count=200):
        settle(fn)
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record()
        for _ in range(count):
            fn()
        last.record()
        torch.cuda.synchronize()
        return round(first.elapsed_time(last) / count * 1e3, 2)

    n = k = 3072
    weights = [(torch.randn(n, k, device="cuda") * 0.02).to(torch.bfloat16) for _ in range(24)]      # 453 MB: more than the 256 MB last-level cache
    rows_out = {}
    for m in (256, 1024, 4096):
        x = torch.randn(m, k, device="cuda").to(torch.bfloat16)
        entry = {}
        for name, product in (("own", lambda w: kernels.gemm_bf16(x, w, None)), ("library", lambda w: F.linear(x, w))):
            turn = [0]

            def rotating():
                turn[0] = (turn[0] + 1) % len(weights)
                return product(weights[turn[0]])

            entry[name] = {"same_weight_us": timed(lambda: product(weights[0])), "rotating_weights_us": timed(rotating)}
        entry["bit_identical_products"] = bool(torch.equal(kernels.gemm_bf16(x, weights[0], None), F.linear(x, weights[0])))
        rows_out[f"M={m}"] = entry
    del weights
    sweep = {}
    for inner in (64, 256, 1024, 2048, 3072, 6144):
        x = torch.randn(4096, inner, device="cuda").to(torch.bfloat16)
        w = (torch.randn(n, inner, device="cuda") * 0.02).to(torch.bfloat16)
        sweep[f"K={inner}"] = {"own_us": timed(lambda: kernels.gemm_bf16(x, w, None)), "library_us": timed(lambda: F.linear(x, w))}
    flops = 2.0 * 4096 * n * k
    own = rows_out["M=4096"]["own"]["rotating_weights_us"]
    result = {
        "metric": "bf16 GEMM TFLOP/s, 4096 x 3072 x 3072, weight from memory", "value": round(flops / own / 1e6, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": 200, "warmup": 0, "ms_per_step": round(own / 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "y = x W^T, N = K = 3072, bf16, f32 accumulation; own kernel (ep_hip_gemm_bf16) beside the vendor library's",
                   "by_rows": rows_out, "by_inner_size_at_M_4096": sweep},
        "roofline": {"bound": "mfma", "achieved": round(flops / own / 1e6, 2), "peak": MFMA_PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / own / 1e6 / MFMA_PEAK_BF16_TFLOPS, 5), "traffic": None},
    }
    print(json.dumps(result))
    return 0


def gemm_phases_workload(args, ep):
    """`--workload gemm_phases [--rows M]`: the N = K = 3072 bf16 product with M activation rows in a fixed dispatch order,
    for counter and trace runs that have to tell the launches apart. For this library's product, then for the vendor
    library's: 4 launches on weight 0, 24 on 24 different weights (untimed), then **16 on weight 0** (launches 28..43 of that
    kernel: operands in the caches), then **24 on the 24 weights in turn** (launches 44..67: the weight comes from memory,
    453 MB of weights pass between two uses of one). Each timed phase sits between one pair of events."""
    from torch.nn import functional as F
    from entropack_amd.linear import kernels
    torch.manual_seed(0)
    weights = [(torch.randn(3072, 3072, device="cuda") * 0.02).to(torch.bfloat16) for _ in range(24)]
    x = torch.randn(args.rows, 3072, device="cuda").to(torch.bfloat16)
    out = {}
    for name, product in (("own", lambda w: kernels.gemm_bf16(x, w, None)), ("library", lambda w: F.linear(x, w))):
        for _ in range(4):
            product(weights[0])
        for w in weights:
            product(w)
        torch.cuda.synchronize()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        marks[0].record()
        for _ in range(16):
            product(weights[0])
        marks[1].record()
        torch.cuda.synchronize()
        marks[2].record()
        for w in weights:
            product(w)
        marks[3].record()
        torch.cuda.synchronize()
        out[name] = {"same_weight_us": round(marks[0].elapsed_time(marks[1]) / 16 * 1e3, 2),
                     "rotating_weights_us": round(marks[2].elapsed_time(marks[3]) / 24 * 1e3, 2)}
    own = out["own"]["rotating_weights_us"]
    flops = 2.0 * args.rows * 3072 * 3072
    print(json.dumps({
        "metric": f"bf16 GEMM TFLOP/s, {args.rows} x 3072 x 3072, weight from memory, clocks not settled", "value": round(flops / own / 1e6, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": 24, "warmup": 28, "ms_per_step": round(own / 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"y = x W^T, M = {args.rows}, N = K = 3072, bf16: 16 launches on one weight, 24 on 24 weights, own then library",
                   "phases": out}}))
    return 0


def fused_lds_workload(args, ep):
    """`--workload fused_lds`: configuration 3's layer (W 3072 x 3072 @ 4 bpp + bias, seed 2) in `fused_through_lds` mode, the
    one kernel in which the matrix cores multiply decoded tiles taken from LDS, beside the two other modes, for M = 16,
    256, 1024 and the configuration's 4096, with the default tiles and with `tile_elements` 4096. Whole forwards, host time
    included; the profile summaries under profiles/ give the kernels on their own."""
    from torch.nn import functional as F
    torch.manual_seed(2)
    dense = torch.nn.Linear(3072, 3072, dtype=torch.bfloat16)
    dense.weight.data.copy_((torch.randn(3072, 3072) * 0.02).to(torch.bfloat16))
    dense.bias.data.copy_((torch.randn(3072) * 0.01).to(torch.bfloat16))
    x = torch.randn(4096, 3072).to(torch.bfloat16).cuda()
    result = {"metric": "CompressedLinear forward, fused decode-to-GEMM through LDS against decode + GEMM", "unit": "ms", "n_gpus": 1,
              "steps": args.steps, "warmup": args.warmup, "higher_is_better": False, "dtype": "bf16", "data": "synthetic",
              "config": {"workload": "CompressedLinear 3072x3072 @ 4.0 bpp + bias, X [M, 3072] bf16, seed 2"}}
    for tile_elements in (None, 4096):
        options = {} if tile_elements is None else {"tile_elements": tile_elements}
        layers = {mode: ep.CompressedLinear.from_linear(dense, config=ep.EntroPackLossyConfig(target_bpp=4.0, **options), forward_mode=mode).cuda()
                  for mode in ("decode_then_gemm", "fused", "fused_through_lds")}
        weight = layers["fused"].dequantize("cuda")
        section = {}
        for m in (16, 256, 1024, 4096):
            part = x[:m].contiguous()
            reference = F.linear(part.double(), weight.double(), dense.bias.data.cuda().double()).float().to(torch.bfloat16).double()
            entry = {}
            for mode, layer in layers.items():
                y = layer(part)
                flops = 2.0 * m * 3072 * 3072
                ms = _median_ms(lambda: layer(part), args.steps, warmup=args.warmup)
                entry[mode] = {"ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 2),
                               "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_PEAK_BF16_TFLOPS, 5),
                               "rel_l2_vs_f64_reference": ((y.double() - reference).norm() / reference.norm()).item()}
            section[f"M={m}"] = entry
        result["default_tiles" if tile_elements is None else f"tile_elements={tile_elements}"] = section
    result["value"] = result["default_tiles"]["M=4096"]["fused_through_lds"]["ms"]
    result["ms_per_step"] = result["value"]
    print(json.dumps(result))
    return 0


def encode_workload(args, ep):
    """The step before the path: `compress` of the target weight (8192 x 28672 bf16, 4.0 bpp) on the device
    (`hip_encode.encode`, kernels `ep_hip_encode_*`), whole call with its host synchronisations, then kernel by kernel
    between events with the clocks settled. Parity: the first 1024 rows encoded by both lanes from the CPU lane's row
    RMS give byte-identical buffers (scales to 1e-5); the full container decodes without an error flag to the rate and
    error the CPU lane's container of the sample has. CPU baseline: this package's CPU encoder (bit-identical to the
    reference's eager lane on the golden containers) on 2048 rows, scaled by rows."""
    from entropack_amd.backends import hip as hip_backend
    from entropack_amd.schemes.lattice_rans import eager, hip_encode
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers, recommended_tile_elements, vector_tile_elements
    rows, cols, sigma, seed, bpp, outliers = WORKLOADS["target"]
    weight = make_weight(rows, cols, sigma, seed, outliers)
    tile_elements = recommended_tile_elements(bpp)
    options = dict(target_bpp=bpp, prob_bits=None, tile_elements=tile_elements)
    on_gpu = weight.cuda()
    hip_encode.encode(weight=on_gpu[:256], **options)                      # loads the library, warms the allocator
    torch.cuda.synchronize()
    walls = []
    for _ in range(3):
        start = time.perf_counter()
        buffers = hip_encode.encode(weight=on_gpu, **options)
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - start)
    wall = sorted(walls)[1]

    # the full container: decodes cleanly, at the rate asked for
    config = ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="hip")
    restored = hip_lane.decode(buffers, shape=(rows, cols), dtype=torch.bfloat16)
    torch.cuda.synchronize()
    hip_lane.check_errors(buffers)
    stored = sum(t.numel() * t.element_size() for t in buffers)
    actual_bpp = 8.0 * stored / (rows * cols)
    error = float((restored.float() - on_gpu.float()).norm() / on_gpu.float().norm())
    del restored

    # parity and CPU baseline on a sample of rows
    sample_rows, cpu_rows = 1024, 2048
    sample = weight[:sample_rows].float().contiguous()
    rms = eager.row_rms(sample, weight.dtype)
    start = time.perf_counter()
    cpu_container = eager.encode(weight=weight[:cpu_rows], **options)
    cpu_seconds = time.perf_counter() - start
    cpu_sample = eager.encode(weight=sample, **options)
    gpu_sample = hip_encode.encode_normalised(sample.cuda(), rms.cuda(), **options)
    identical = all(torch.equal(a.cpu(), b) for key, a, b in zip(LatticeBuffers._fields, gpu_sample, cpu_sample) if key != "scales")
    scales_close = bool(torch.allclose(gpu_sample.scales.cpu(), cpu_sample.scales, rtol=1e-5, atol=0.0))
    cpu_dense = ep.decompress(ep.compress(weight[:cpu_rows], ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager")).to("cuda"), config)
    cpu_error = float((cpu_dense.float() - on_gpu[:cpu_rows].float()).norm() / on_gpu[:cpu_rows].float().norm())
    cpu_bpp = 8.0 * sum(t.numel() * t.element_size() for t in cpu_container) / (cpu_rows * cols)
    parity = identical and scales_close and abs(actual_bpp - cpu_bpp) <= 0.01 * cpu_bpp and abs(error - cpu_error) <= 0.01 * cpu_error

    # kernel by kernel
    library, stream = hip_backend.library(), torch.cuda.current_stream().cuda_stream
    x = on_gpu.float().contiguous()
    quantizer = hip_encode.DeviceQuantizer(x, hip_encode.row_rms(x, weight.dtype))
    scale = eager.bisect_scale(quantizer, bpp, 11, tile_elements, 12, 262144)
    q = quantizer.quantize(scale)
    stats = q.stats()
    meta, freq_all, cdf_all = eager.stream_tables(stats, q.histograms(stats), 11)
    vectors, tile_vectors = q.vectors, vector_tile_elements(tile_elements)
    tiles = (vectors + tile_vectors - 1) // tile_vectors

    def timed(fn, count=20):
        settle(fn, 0.1)
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record()
        for _ in range(count):
            fn()
        last.record()
        torch.cuda.synchronize()
        return first.elapsed_time(last) / count * 1e3

    def check(status):
        if status:
            raise hip_backend.HipError("ep_hip_encode", status, "")

    summary = torch.empty(33, dtype=torch.int64, device="cuda")
    alphabets = np.where(stats[:, 0] > 0, stats[:, 2] - stats[:, 1] + 1, 0)
    starts = np.concatenate([[0], np.cumsum(alphabets)]).astype(np.int64)
    bin_rel = torch.from_numpy((starts[:17] - stats[:, 1]).astype(np.int32)).cuda()
    bins = torch.empty(int(starts[-1]), dtype=torch.int64, device="cuda")
    scales = torch.empty(rows, dtype=torch.float32, device="cuda")
    entries = hip_encode.table_entries(freq_all, cdf_all).cuda()
    table_rel = torch.from_numpy((meta[:, 2] - meta[:, 1]).astype(np.int32)).cuda()
    states = torch.empty((tiles, 32), dtype=torch.int32, device="cuda")
    tile_words = torch.empty(tiles, dtype=torch.int32, device="cuda")
    scratch = torch.empty(tiles * tile_vectors * 9, dtype=torch.int16, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    offsets = torch.empty(tiles + 1, dtype=torch.int32, device="cuda")
    total = torch.empty(1, dtype=torch.int64, device="cuda")
    kernels = {}
    kernels["quantize"] = (timed(lambda: check(library.ep_hip_encode_quantize(
        x.data_ptr(), quantizer.rms.data_ptr(), cols, scale, 0, rows, q.coset.data_ptr(), q.fields.data_ptr(), summary.data_ptr(), stream))),
        4 * rows * cols + 33 * vectors)
    kernels["histogram"] = (timed(lambda: check(library.ep_hip_encode_histogram(
        q.coset.data_ptr(), q.fields.data_ptr(), vectors, bin_rel.data_ptr(), bins.numel(), bins.data_ptr(), stream))), 33 * vectors)
    kernels["row_scales"] = (timed(lambda: check(library.ep_hip_encode_row_scales(
        x.data_ptr(), quantizer.rms.data_ptr(), cols, scale, rows, q.coset.data_ptr(), q.fields.data_ptr(), scales.data_ptr(), 0, stream))),
        4 * rows * cols + 33 * vectors)
    kernels["rans"] = (timed(lambda: check(library.ep_hip_encode_rans(
        q.coset.data_ptr(), q.fields.data_ptr(), vectors, entries.data_ptr(), table_rel.data_ptr(), entries.numel(), 11, tile_vectors,
        states.data_ptr(), tile_words.data_ptr(), scratch.data_ptr(), flag.data_ptr(), stream))), None)
    check(library.ep_hip_encode_offsets(tile_words.data_ptr(), tiles, offsets.data_ptr(), total.data_ptr(), stream))
    words = int(total.item())
    kernels["rans"] = (kernels["rans"][0], 33 * vectors + 2 * words + 132 * tiles)
    payload = torch.empty(words, dtype=torch.int16, device="cuda")
    kernels["offsets"] = (timed(lambda: check(library.ep_hip_encode_offsets(
        tile_words.data_ptr(), tiles, offsets.data_ptr(), total.data_ptr(), stream))), 8 * tiles)
    kernels["gather"] = (timed(lambda: check(library.ep_hip_encode_gather(
        scratch.data_ptr(), offsets.data_ptr(), tiles, tile_vectors * 9, payload.data_ptr(), stream))), 4 * words)
    assert int(flag.item()) == 0
    by_kernel = {name: {"us": round(us, 1), "algorithmic_bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1)} for name, (us, nbytes) in kernels.items()}
    dominant = max(kernels, key=lambda name: kernels[name][0])
    us, nbytes = kernels[dominant]
    weights = rows * cols
    result = {
        "metric": "lattice_rans encode, weights per second (whole compress call on the device)", "value": round(weights / wall / 1e9, 3),
        "unit": "Gweights/s", "n_gpus": 1, "steps": 3, "warmup": 1, "ms_per_step": round(wall * 1e3, 2), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32/f64 quantise, u32 rANS", "data": "synthetic",
        "config": {"workload": f"compress {rows}x{cols} bf16 N(0,{sigma}) seed {seed} @ {bpp} bpp on the device (12 search iterations on a "
                               "row subsample, full quantise, histograms, refit, rANS encode, gather)",
                   "actual_bpp": round(actual_bpp, 4), "relative_error": round(error, 5), "lattice_scale": round(scale, 6), "kernels_sum_ms": round(sum(v[0] for v in kernels.values()) / 1e3, 3),
                   "by_kernel": by_kernel, "sample_identical_to_cpu_lane": identical, "sample_scales_within_1e-5": scales_close,
                   "cpu_lane_on_sample": {"rows": cpu_rows, "actual_bpp": round(cpu_bpp, 4), "relative_error": round(cpu_error, 5)}},
        "parity": parity,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": round(nbytes / us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 5), "traffic": None},
        "cpu_baseline": {"value": round(cpu_rows * cols / cpu_seconds / 1e9, 4), "unit": "Gweights/s", "cores": eager._threads(), "kind": "port",
                         "sample": f"first {cpu_rows} of {rows} rows through this package's CPU encoder (bit-identical to the reference's eager "
                                   f"lane on its golden containers), {cpu_seconds:.2f} s"},
    }
    print(json.dumps(result))
    return 0 if parity else 1


def lossless_encode_workload(args, ep):
    """`compress` of the 8192 x 28672 bf16 weight with the lossless tile_ans scheme on the device (default options: 8192
    elements per tile, automatic precision; low byte raw, high byte coded): whole call, then kernel by kernel between
    events. Parity: the first 2048 rows give the CPU lane's container byte for byte, and the full container decodes to
    the input. CPU baseline: this package's CPU encoder on those rows (byte-identical to the reference's on its golden
    containers), scaled by rows."""
    from entropack_amd.backends import hip as hip_backend
    from entropack_amd.schemes.lattice_rans.hip_encode import table_entries
    from entropack_amd.schemes.tile_ans import eager as tile_eager
    from entropack_amd.schemes.tile_ans.format import TileBuffers, num_tiles
    rows, cols, sigma, seed = 8192, 28672, 0.015, 4
    weight = make_weight(rows, cols, sigma, seed, False)
    on_gpu = weight.cuda()
    config = ep.TileANSConfig(execution_backend="hip")
    ep.compress(on_gpu[:64], config)
    torch.cuda.synchronize()
    walls = []
    for _ in range(3):
        start = time.perf_counter()
        container = ep.compress(on_gpu, config)
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - start)
    wall = sorted(walls)[1]
    lossless = bool(torch.equal(ep.decompress(container, ep.TileANSConfig()).view(torch.int16), on_gpu.view(torch.int16)))
    stored = sum(t.numel() * t.element_size() for t in container.buffers.values())

    cpu_rows = 2048
    start = time.perf_counter()
    on_cpu = ep.compress(weight[:cpu_rows], ep.TileANSConfig(execution_backend="eager"))
    cpu_seconds = time.perf_counter() - start
    sample = ep.compress(on_gpu[:cpu_rows], config)
    identical = all(torch.equal(sample.buffers[key].cpu(), on_cpu.buffers[key]) for key in TileBuffers._fields)

    library, stream = hip_backend.library(), torch.cuda.current_stream().cuda_stream
    tile_elements, prob_bits, num_lanes, num_elements = (int(v) for v in container.buffers["layout"].tolist())
    counts_device = torch.empty((num_lanes, 256), dtype=torch.int64, device="cuda")

    def check(status):
        if status:
            raise hip_backend.HipError("ep_hip_tile_ans", status, "")

    def timed(fn, count=20):
        settle(fn, 0.1)
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record()
        for _ in range(count):
            fn()
        last.record()
        torch.cuda.synchronize()
        return first.elapsed_time(last) / count * 1e3

    nbytes = num_elements * num_lanes
    kernels = {"histogram": (timed(lambda: check(library.ep_hip_tile_ans_histogram(on_gpu.data_ptr(), num_elements, num_lanes, counts_device.data_ptr(), stream))), nbytes)}
    _, freq, cdfs, _, modes = tile_eager.coding_plan(counts_device.cpu().numpy(), prob_bits, 7.9, tile_elements)
    tiles = num_tiles(num_elements, tile_elements)
    streams, coded = tiles * num_lanes, int((modes == 0).sum())
    entries = table_entries(freq.astype(np.int64).reshape(-1), cdfs.astype(np.int64).reshape(-1)).cuda()
    raw_flags = np.ascontiguousarray(modes != 0, dtype=np.uint8)
    states = torch.empty((tiles * coded, 32), dtype=torch.int32, device="cuda")
    stream_words = torch.empty(streams, dtype=torch.int32, device="cuda")
    scratch = torch.empty(streams * tile_elements, dtype=torch.int16, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    offsets = torch.empty(streams + 1, dtype=torch.int32, device="cuda")
    total = torch.empty(1, dtype=torch.int64, device="cuda")
    words = container.buffers["payload"].numel()
    payload = torch.empty(words, dtype=torch.int16, device="cuda")
    kernels["encode"] = (timed(lambda: check(library.ep_hip_tile_ans_encode(
        on_gpu.data_ptr(), num_elements, num_lanes, tile_elements, prob_bits, entries.data_ptr(), raw_flags.ctypes.data, states.data_ptr(),
        stream_words.data_ptr(), scratch.data_ptr(), tile_elements, flag.data_ptr(), stream))), nbytes + 2 * words + 128 * tiles * coded)
    kernels["offsets"] = (timed(lambda: check(library.ep_hip_encode_offsets(stream_words.data_ptr(), streams, offsets.data_ptr(), total.data_ptr(), stream))), 8 * streams)
    kernels["gather"] = (timed(lambda: check(library.ep_hip_encode_gather(scratch.data_ptr(), offsets.data_ptr(), streams, tile_elements, payload.data_ptr(), stream))), 4 * words)
    assert int(flag.item()) == 0 and int(total.item()) == words
    by_kernel = {name: {"us": round(us, 1), "algorithmic_bytes": b, "GBps": round(b / us / 1e3, 1)} for name, (us, b) in kernels.items()}
    dominant = max(kernels, key=lambda name: kernels[name][0])
    us, b = kernels[dominant]
    parity = lossless and identical
    result = {
        "metric": "tile_ans encode, input GB/s (whole compress call on the device)", "value": round(nbytes / wall / 1e9, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": 3, "warmup": 1, "ms_per_step": round(wall * 1e3, 2), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8 symbols, u32 rANS", "data": "synthetic",
        "config": {"workload": f"lossless compress {rows}x{cols} bf16 N(0,{sigma}) seed {seed} on the device, default options "
                               f"(tile_elements {tile_elements}, probability_bits {prob_bits}, lane modes {modes.tolist()})",
                   "stored_over_input": round(stored / nbytes, 4), "kernels_sum_ms": round(sum(v[0] for v in kernels.values()) / 1e3, 3),
                   "by_kernel": by_kernel, "sample_identical_to_cpu_lane": identical, "lossless": lossless},
        "parity": parity,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": round(b / us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 5), "traffic": None},
        "cpu_baseline": {"value": round(cpu_rows * cols * 2 / cpu_seconds / 1e9, 4), "unit": "GB/s", "cores": tile_eager._threads(), "kind": "port",
                         "sample": f"first {cpu_rows} of {rows} rows through this package's CPU encoder, {cpu_seconds:.2f} s"},
    }
    print(json.dumps(result))
    return 0 if parity else 1


def copy_probe(args, device):
    """One plain device copy of `--copy-probe-mib` MiB: the calibration of the FETCH_SIZE / WRITE_SIZE counters."""
    if args.copy_probe_mib:
        probe = torch.empty(args.copy_probe_mib << 20, dtype=torch.uint8, device=device)
        probe.zero_()
        torch.empty_like(probe).copy_(probe)          # reads and writes exactly copy_probe_mib MiB
        torch.cuda.synchronize()
        del probe


def lossless_workload(args, ep):
    """The lossless neighbour of the target: tile_ans decode of 8192 x 28672 bf16 N(0, 0.015) seed 4 (the reference's
    default options for bfloat16: 8192-element tiles, 10-bit tables; low byte raw, high byte coded)."""
    from entropack_amd.schemes.base import packed_buffers
    from entropack_amd.schemes.tile_ans import hip as tile_lane
    from entropack_amd.schemes.tile_ans.format import TileBuffers
    rows, cols, sigma, seed = 8192, 28672, 0.015, 4
    started = time.perf_counter()
    weight = make_weight(rows, cols, sigma, seed, False)
    container = ep.compress(weight, ep.TileANSConfig(execution_backend="eager"))
    encode_seconds = time.perf_counter() - started
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    on_gpu = container.to(device)
    buffers = packed_buffers(on_gpu.buffers, TileBuffers)
    alg_bytes = sum(t.numel() * t.element_size() for t in container.buffers.values()) + rows * cols * 2

    def step():
        return tile_lane.decode(buffers, dtype=torch.bfloat16)

    copy_probe(args, device)
    dense = step()
    settle(step)
    for _ in range(max(args.warmup, 1)):
        dense = step()
    torch.cuda.synchronize()
    tile_lane.check_errors(buffers)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall = time.perf_counter()
    first.record()
    for _ in range(args.steps):
        dense = step()
    last.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - wall) / args.steps
    kernel_avg_ms = first.elapsed_time(last) / args.steps
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for begin, end in events:
        begin.record()
        dense = step()
        end.record()
    torch.cuda.synchronize()
    kernel_ms = sorted(begin.elapsed_time(end) for begin, end in events)
    # The same launches rotating through device copies of the container: none finds its bytes in the last-level cache.
    copies = max(2, -(-ROTATING_INPUT_BYTES // max(1, alg_bytes - rows * cols * 2)))
    rotation = [on_gpu] + [container.to(device) for _ in range(copies - 1)]
    rotating = [packed_buffers(one.buffers, TileBuffers) for one in rotation]
    turn = [0]

    def rotating_step():
        turn[0] = (turn[0] + 1) % len(rotating)
        return tile_lane.decode(rotating[turn[0]], dtype=torch.bfloat16)

    for _ in rotating:
        rotating_step()
    settle(rotating_step)
    torch.cuda.synchronize()
    first_rotating, last_rotating = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first_rotating.record()
    for _ in range(args.steps):
        rotating_step()
    last_rotating.record()
    torch.cuda.synchronize()
    rotating_ms = first_rotating.elapsed_time(last_rotating) / args.steps
    for one in rotating:
        tile_lane.check_errors(one)
    del rotation, rotating
    tile_elements, prob_bits, lanes, elements = (int(v) for v in container.buffers["layout"].tolist())
    result = {
        "metric": "lossless decode GB/s (+% HBM roofline)", "value": round(alg_bytes / wall / 1e9, 3), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {
            "workload": f"tile_ans decode to bf16, {rows}x{cols} N(0,{sigma}) seed {seed}, default options",
            "tile_elements": tile_elements, "prob_bits": prob_bits, "lane_modes": container.buffers["lane_modes"].tolist(),
            "stored_over_dense": round(container.storage_nbytes() / (rows * cols * 2), 4), "algorithmic_bytes": alg_bytes,
            "elements_per_s": round(rows * cols / wall, 1), "encode_seconds_cpu": round(encode_seconds, 2),
            "lossless": bool(torch.equal(dense.view(torch.int16).reshape(rows, cols).cpu(), weight.view(torch.int16))),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(alg_bytes / (kernel_avg_ms * 1e-3) / 1e9, 3), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(alg_bytes / (kernel_avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5), "traffic": measured_traffic("tile_ans")[0],
            "traffic_source": measured_traffic("tile_ans")[1],
            "kernel_ms_avg": round(kernel_avg_ms, 5), "kernel_ms_median": round(kernel_ms[len(kernel_ms) // 2], 5),
            "kernel_ms_avg_rotating_inputs": round(rotating_ms, 5),
            "frac_rotating_inputs": round(alg_bytes / (rotating_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5),
            "inputs": f"kernel_ms_avg: the same container every launch; rotating inputs: {copies} device copies of it in turn "
                      "(each launch reads its container from memory, not from the 256 MB last-level cache)",
        },
    }
    if not args.no_cpu:
        from oracle import c_oracle
        c_oracle.load_tile_ans()
        host = host_arrays(container.buffers)
        threads = min(16, os.cpu_count() or 1)
        best = float("inf")
        for _ in range(2):
            begin = time.perf_counter()
            expect = c_oracle.tile_ans_decode(host, 2, threads=threads)
            best = min(best, time.perf_counter() - begin)
        result["cpu_baseline"] = {
            "value": round(alg_bytes / best / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"whole container, C port of the reference CPU decoder, {threads} OpenMP threads, best of 2, {best:.3f} s"}
        result["config"]["bit_exact_vs_oracle"] = bool(np.array_equal(dense.view(torch.uint8).cpu().numpy().reshape(-1), expect))
    print(json.dumps(result))
    return 0 if parity_holds(result) else 1


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--workload", default="target", choices=sorted(WORKLOADS) + ["c4", "tile_ans", "gemm", "gemm_phases", "fused_lds", "encode", "tile_ans_encode"])
    parser.add_argument("--rows", type=int, default=256, help="activation rows of the gemm_phases workload")
    parser.add_argument("--stack-blocks", type=int, default=30, help="blocks of the c4 layer stack (30 = the full 120 layers)")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the parity check")
    parser.add_argument("--no-linear", action="store_true", help="skip the CompressedLinear (config 3) section")
    parser.add_argument("--no-configs", action="store_true", help="skip the decode_configs section (c2, c5a, c5b, c4) of the default run")
    parser.add_argument("--copy-probe-mib", type=int, default=0,
                        help="also run one plain device copy of this many MiB (calibrates FETCH_SIZE / WRITE_SIZE counters)")
    parser.add_argument("--prob-bits", type=int, default=None, help="encode with this prob_bits instead of the rate's default")
    parser.add_argument("--table-kind", type=int, default=None, help="force an ep_hip_table_kind (debugging)")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X; this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import entropack_amd as ep
    from entropack_amd.schemes.lattice_rans import hip as hip_lane
    from entropack_amd.schemes.lattice_rans.format import LatticeBuffers

    if args.workload == "c4":
        return stack_workload(args, ep)
    if args.workload == "tile_ans":
        return lossless_workload(args, ep)
    if args.workload == "gemm":
        return gemm_workload(args, ep)
    if args.workload == "gemm_phases":
        return gemm_phases_workload(args, ep)
    if args.workload == "fused_lds":
        return fused_lds_workload(args, ep)
    if args.workload == "encode":
        return encode_workload(args, ep)
    if args.workload == "tile_ans_encode":
        return lossless_encode_workload(args, ep)
    rows, cols, sigma, seed, bpp, outliers = WORKLOADS[args.workload]
    started = time.perf_counter()
    weight = make_weight(rows, cols, sigma, seed, outliers)
    config = ep.EntroPackLossyConfig(target_bpp=bpp, execution_backend="eager", prob_bits=args.prob_bits)
    container = ep.compress(weight, config)
    encode_seconds = time.perf_counter() - started
    del weight

    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    hip_lane.FORCE_TABLE_KIND = args.table_kind
    on_gpu = container.to(device)
    lattice = LatticeBuffers(**{key: on_gpu.buffers[key] for key in LatticeBuffers._fields})
    cols_padded = int(container.buffers["layout"][0])
    alg_bytes = algorithmic_bytes(container.buffers, rows, cols_padded, 2)

    # Every launch of the timed region reads its container from memory, as a model that decodes each layer once per
    # forward does: the steps rotate through enough device copies of the container that none of them is still in the
    # card's 256 MB last-level cache when its turn comes again. (One container decoded over and over keeps its compressed
    # bytes there; that figure is reported beside, as `same_container`.)
    copies = max(2, -(-ROTATING_INPUT_BYTES // max(1, alg_bytes - 2 * rows * cols_padded)))
    rotation = [on_gpu] + [container.to(device) for _ in range(copies - 1)]
    rotating = [LatticeBuffers(**{key: one.buffers[key] for key in LatticeBuffers._fields}) for one in rotation]
    turn = [0]

    def step():
        turn[0] = (turn[0] + 1) % len(rotating)
        return hip_lane.decode(rotating[turn[0]], shape=(rows, cols), dtype=torch.bfloat16)

    def same_container_step():
        return hip_lane.decode(lattice, shape=(rows, cols), dtype=torch.bfloat16)

    copy_probe(args, device)

    # From idle first (the device has done nothing while the host encoded): `warmup` + `steps` launches as they come.
    for _ in rotating:
        dense = step()                                # builds the plans
    torch.cuda.synchronize()
    for one in rotating:
        hip_lane.check_errors(one)
    time.sleep(0.2)
    for _ in range(max(args.warmup, 1)):
        dense = step()
    idle_first, idle_last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    idle_first.record()
    for _ in range(args.steps):
        dense = step()
    idle_last.record()
    torch.cuda.synchronize()
    from_idle_ms = idle_first.elapsed_time(idle_last) / args.steps
    # Then with the clocks settled: SETTLE_SECONDS of the same launches, the warm-up steps, the timed steps.
    settle(step)
    for _ in range(max(args.warmup, 1)):
        dense = step()
    torch.cuda.synchronize()

    # The timed region: exactly `steps` launches back to back between two synchronisations, with one pair of HIP events
    # on the launch stream around all of them (average launch duration = their distance / steps; events between the
    # launches would put a marker packet, and a few microseconds, between every two kernels).
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    wall = time.perf_counter()
    first.record()
    for _ in range(args.steps):
        dense = step()
    last.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall
    kernel_avg_ms = first.elapsed_time(last) / args.steps
    ms_per_step = wall * 1e3 / args.steps
    # Outside the timed region: the same launches bracketed one by one, for the spread.
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for begin, end in events:
        begin.record()
        dense = step()
        end.record()
    torch.cuda.synchronize()
    kernel_ms = sorted(begin.elapsed_time(end) for begin, end in events)
    for one in rotating:
        hip_lane.check_errors(one)
    dense = same_container_step()                     # the tensor the oracle check below compares
    del rotation, rotating

    # The same launches on one container over and over: its compressed bytes stay in the last-level cache.
    settle(same_container_step)
    torch.cuda.synchronize()
    first_same, last_same = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first_same.record()
    for _ in range(args.steps):
        same_container_step()
    last_same.record()
    torch.cuda.synchronize()
    same_ms = first_same.elapsed_time(last_same) / args.steps
    hip_lane.check_errors(lattice)

    result = {
        "metric": "lossy decode GB/s (+% HBM roofline); CompressedLinear TFLOPS @ M=4096, 4 bpp",
        "value": round(alg_bytes / (wall / args.steps) / 1e9, 3),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u32",
        "data": "synthetic",
        "config": {
            "workload": f"lattice_rans decode to bf16, {rows}x{cols} N(0,{sigma}) seed {seed}"
                        f"{' +0.1% x20 outliers' if outliers else ''} @ {bpp} bpp target",
            "actual_bpp": round(container.actual_bpp, 4), "tiles": int(lattice.states.shape[0]),
            "prob_bits": int(container.buffers["layout"][1]), "tile_elements": int(container.buffers["layout"][2]),
            "table_kind": hip_lane.launch_table_kind(lattice, shape=(rows, cols), dtype=torch.bfloat16), "algorithmic_bytes": alg_bytes,
            "params_per_s": round(rows * cols / (wall / args.steps), 1), "encode_seconds_cpu": round(encode_seconds, 2),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(alg_bytes / (kernel_avg_ms * 1e-3) / 1e9, 3), "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": round(alg_bytes / (kernel_avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5),
            "traffic": measured_traffic(args.workload, args.table_kind)[0], "traffic_source": measured_traffic(args.workload, args.table_kind)[1],
            "kernel_ms_avg": round(kernel_avg_ms, 5), "kernel_ms_median": round(kernel_ms[len(kernel_ms) // 2], 5),
            "kernel_ms_min": round(kernel_ms[0], 5),
            "kernel_ms_avg_from_idle": round(from_idle_ms, 5),
            "frac_from_idle": round(alg_bytes / (from_idle_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5),
            "kernel_ms_avg_same_container": round(same_ms, 5),
            "frac_same_container": round(alg_bytes / (same_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5),
            "inputs": f"timed region: {copies} device copies of the container in turn, so that each launch reads its container "
                      f"from memory; same_container: one container every launch (its compressed bytes stay in the 256 MB last-level cache)",
            "clocks": f"settled: {SETTLE_SECONDS} s of untimed launches of the same kernel before the warm-up steps; "
                      f"from idle = the first {args.warmup} + {args.steps} launches after 0.2 s without work",
        },
    }

    if not args.no_linear:
        result["linear"] = linear_section(ep, args.steps)
        result["linear_stack"] = stack_linear_section(ep, args.steps)
        result["linear_int8"] = int8_linear_section(ep, args.steps)
        if rows * cols >= 1 << 27:
            result["linear_small_m"] = small_m_section(ep, on_gpu, rows, cols, bpp, args.steps)

    if not args.no_cpu:
        host = host_arrays(container.buffers)
        threads = min(16, os.cpu_count() or 1)
        expect, baseline = cpu_baseline(host, rows, cols_padded, alg_bytes, threads)
        result["cpu_baseline"] = baseline
        result["cpu_python_loop"] = python_loop_baseline(host, rows, cols_padded, alg_bytes)
        got = dense.view(torch.int16).cpu().numpy().view(np.uint16)
        result["config"]["bit_exact_vs_oracle"] = bool(np.array_equal(got, expect[:, :cols]))
        del host, expect, got
    del dense
    if args.workload == "target" and not args.no_configs:
        # The other decode configurations of the benchmark, each on its own container, checked like the headline.
        del on_gpu, lattice, container
        torch.cuda.empty_cache()
        configs = {}
        for name in ("c2", "c5a", "c5b"):
            configs[name] = decode_case(ep, name, max(10, args.steps // 2), args.warmup, not args.no_cpu,
                                        small_m=name in ("c5a", "c5b") and not args.no_linear)
            torch.cuda.empty_cache()
        configs["c4"] = stack_case(ep, args.steps, not args.no_cpu)
        result["decode_configs"] = configs
    print(json.dumps(result))
    return 0 if parity_holds(result) else 1


def parity_holds(node):
    """False when any `bit_exact...` / `identical...` / `lossless` flag anywhere in a result is false."""
    if isinstance(node, dict):
        for key, value in node.items():
            if isinstance(value, bool) and (key.startswith("bit_exact") or key.startswith("identical") or key == "lossless") and not value:
                print(f"bench.py: parity check failed: {key}", file=sys.stderr)
                return False
            if not parity_holds(value):
                return False
    return True


if __name__ == "__main__":
    sys.exit(main())
