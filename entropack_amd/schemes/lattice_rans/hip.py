"""`hip` lane of lattice_rans: decode (and encode, hip_encode.py) on an MI355X through the C ABI of libentropack_hip.so.

Module-level `decode(buffers, *, shape, dtype, threads_per_block, l2_prefetch)` is the lane contract of the
reference's CUDA lane (entropack/schemes/lattice_rans/cuda.py:781-805): all buffers on the device, result
`[rows, padded cols]` of `dtype` on the same device, enqueued on torch's current stream without a host
synchronisation after the launch. Derived decode tables live in a plan cached on the `layout` tensor object and keyed
by the data pointers it was built from (cuda.py:697-741); the tables themselves are built by a device kernel.

There is no CPU path in this module and no fallback: a missing library or device raises.
"""
import ctypes
import weakref
from dataclasses import dataclass

import numpy as np
import torch

from ...backends import hip as _hip
from ..base import host_copy
from .format import LatticeBuffers, decode_geometry, snap_to_container

#: float8 formats without a store kernel are decoded to float32 and cast on the device, as the reference does.
_VIA_FLOAT32 = frozenset({torch.float8_e4m3fnuz, torch.float8_e5m2fnuz})

#: Test hook: force one ep_hip_table_kind for every new plan (None = let the library choose).
FORCE_TABLE_KIND: int | None = None


@dataclass
class DecodePlan:
    desc: _hip.PlanDesc
    tables: torch.Tensor          # uint8, device; header + slot tables
    error: torch.Tensor           # int32[1], device; first decode error of any launch using this plan
    key: tuple

    @property
    def table_kind(self) -> str:
        return _hip.TABLE_KIND_NAMES[self.desc.table_kind]


_ERROR_WORDS_PER_POOL = 1024
_error_pools: dict = {}        # device -> [int32 tensor of zeros, words handed out]


def _error_word(device: torch.device) -> torch.Tensor:
    """A zeroed int32[1] for one plan's decode errors, cut from a pool per device: one fill kernel per 1024 plans instead
    of one per plan (a model's containers are planned in a burst when it is first decoded)."""
    pool = _error_pools.get(device)
    if pool is None or pool[1] == _ERROR_WORDS_PER_POOL:
        pool = _error_pools[device] = [torch.zeros(_ERROR_WORDS_PER_POOL, dtype=torch.int32, device=device), 0]
    word = pool[0][pool[1]:pool[1] + 1]
    pool[1] += 1
    return word


def _plan_for(buffers: LatticeBuffers, info: dict) -> DecodePlan:
    layout, meta, freq = buffers.layout, buffers.stream_meta, buffers.freq_tables
    device = meta.device
    key = (meta.data_ptr(), freq.data_ptr(), device, FORCE_TABLE_KIND)
    plan = getattr(layout, "_lattice_rans_hip_plan", None)
    if plan is not None and plan.key == key:
        return plan

    lib = _hip.library()
    # Host values of the two small tables: the copies that came with the container, else one small read-back each.
    meta_host = np.ascontiguousarray(host_copy(meta).numpy(), dtype=np.int32)
    freq_host = np.ascontiguousarray(host_copy(freq).view(torch.int16).numpy()).view(np.uint16)
    if meta_host.shape != (17, 4):
        raise ValueError(f"lattice_rans stream_meta must be (17, 4), got {meta_host.shape}")
    desc = _hip.PlanDesc()
    caps = _hip.device_info(device.index if device.index is not None else torch.cuda.current_device())
    status = lib.ep_hip_plan_describe(
        meta_host.ctypes.data, freq_host.ctypes.data if freq_host.size else None, freq_host.size, info["prob_bits"],
        info["tile_elements"], caps.lds_bytes_per_block, -1 if FORCE_TABLE_KIND is None else FORCE_TABLE_KIND, ctypes.byref(desc))
    if status == _hip.EINVAL:
        raise ValueError("lattice_rans stream_meta / freq_tables are inconsistent (ranges, sums or coset stream)")
    _hip.check("ep_hip_plan_describe", status)
    tables = torch.empty(desc.table_bytes, dtype=torch.uint8, device=device)
    error = _error_word(device)
    _hip.check("ep_hip_plan_build", lib.ep_hip_plan_build(
        meta.data_ptr(), _hip.pointer(freq), ctypes.byref(desc), tables.data_ptr(), _hip.current_stream(device)))
    plan = DecodePlan(desc=desc, tables=tables, error=error, key=key)
    layout._lattice_rans_hip_plan = plan
    return plan


_C_INT_MAX = 2 ** 31 - 1


def _check_abi_ranges(info: dict) -> None:
    """The C ABI takes `tile_elements` as a C int. A container's layout holds it as int64, and ctypes would truncate a
    larger value silently: the library would then derive other tiles than the ones the buffers were checked against."""
    if not 0 < info["tile_elements"] <= _C_INT_MAX:
        raise ValueError(f"lattice_rans tile_elements {info['tile_elements']} is outside what the hip lane takes (1 .. 2**31 - 1)")


def _checked_geometry(buffers: LatticeBuffers, shape, dtype):
    """(geometry, dtype the kernel stores, decoded via float32?) of one container, after the lane's argument checks."""
    device = buffers.payload.device
    if device.type != "cuda":
        raise RuntimeError(f"the hip lane decodes device buffers only, got {device}")
    info = decode_geometry(buffers._asdict(), shape)
    _check_abi_ranges(info)
    if buffers.scales.numel() != info["rows"] or buffers.states.numel() != max(1, info["total_tiles"]) * 32 \
            or buffers.offsets.numel() != max(1, info["total_tiles"]) + 1:
        raise ValueError("lattice_rans buffers do not match the container geometry")
    for tensor in buffers:
        if not tensor.is_contiguous():
            raise ValueError("lattice_rans buffers must be contiguous")
    via_float32 = dtype in _VIA_FLOAT32
    out_dtype = torch.float32 if via_float32 else dtype
    if out_dtype not in _hip.STORE_KINDS:
        raise ValueError(f"lattice_rans does not support output dtype {dtype}")
    return info, out_dtype, via_float32


class _PreparedDecode:
    """Everything one container's decode call needs except the output and the stream, checked once and kept on the
    container's `layout` tensor: the second and later decodes of a container skip the geometry checks, the plan lookup
    and the conversion of a dozen arguments (which together cost more host time than a small layer's kernel runs).

    The object lives on the `layout` tensor, so it refers to the container's tensors weakly: a strong reference would
    close a cycle (layout -> cache -> prepared call -> layout) and a dropped container would keep its device memory until
    the cycle collector runs."""

    __slots__ = ("tensors", "pointers", "shape", "dtype", "out_dtype", "via_float32", "rows", "cols", "device", "index",
                 "plan", "call", "head", "tail")

    def __init__(self, buffers: LatticeBuffers, shape, dtype):
        info, out_dtype, via_float32 = _checked_geometry(buffers, shape, dtype)
        device = buffers.payload.device
        with torch.cuda.device(device):
            plan = _plan_for(buffers, info)
        self.tensors = tuple(weakref.ref(tensor) for tensor in buffers)
        self.pointers = tuple(tensor.data_ptr() for tensor in buffers)
        self.shape, self.dtype, self.out_dtype, self.via_float32 = tuple(shape), dtype, out_dtype, via_float32
        self.rows, self.cols = info["rows"], info["cols"]
        self.device = device
        self.index = device.index if device.index is not None else torch.cuda.current_device()
        self.plan = plan
        self.call = _hip.library().ep_hip_decode_lattice
        self.head = (_hip.pointer(buffers.payload), buffers.payload.numel(), buffers.offsets.data_ptr(), buffers.states.data_ptr(),
                     buffers.scales.data_ptr(), plan.tables.data_ptr(), ctypes.byref(plan.desc))
        self.tail = (_hip.STORE_KINDS[out_dtype], self.rows, self.cols, info["tile_elements"], plan.error.data_ptr())

    def serves(self, buffers: LatticeBuffers, shape, dtype) -> bool:
        """The same tensor objects at the same addresses, with the plan still theirs."""
        for tensor, held, address in zip(buffers, self.tensors, self.pointers):
            if held() is not tensor or tensor.data_ptr() != address:
                return False
        return getattr(buffers.layout, "_lattice_rans_hip_plan", None) is self.plan and self.plan.key[3] == FORCE_TABLE_KIND

    def run(self) -> torch.Tensor:
        out = torch.empty((self.rows, self.cols), dtype=self.out_dtype, device=self.device)
        if torch.cuda.current_device() == self.index:
            status = self.call(*self.head, out.data_ptr(), *self.tail, torch._C._cuda_getCurrentRawStream(self.index))
        else:
            with torch.cuda.device(self.device):
                status = self.call(*self.head, out.data_ptr(), *self.tail, torch._C._cuda_getCurrentRawStream(self.index))
        if status:
            _hip.check("ep_hip_decode_lattice", status)
        return snap_to_container(out, self.dtype) if self.via_float32 else out


def decode(buffers: LatticeBuffers, *, shape, dtype, threads_per_block=None, l2_prefetch=True) -> torch.Tensor:
    calls = getattr(buffers.layout, "_lattice_rans_hip_calls", None)
    if calls is None:
        calls = buffers.layout._lattice_rans_hip_calls = {}
    key = (dtype, tuple(shape))
    prepared = calls.get(key)
    if prepared is None or not prepared.serves(buffers, shape, dtype):
        prepared = calls[key] = _PreparedDecode(buffers, shape, dtype)
    return prepared.run()


def _job_of(buffers: LatticeBuffers, info: dict, plan: DecodePlan, store_kind: int, out_offset: int = 0) -> "_hip.DecodeJob":
    job = _hip.DecodeJob()
    job.payload_dev = _hip.pointer(buffers.payload)
    job.payload_words = buffers.payload.numel()
    job.offsets_dev = buffers.offsets.data_ptr()
    job.states_dev = buffers.states.data_ptr()
    job.scales_dev = buffers.scales.data_ptr()
    job.tables_dev = plan.tables.data_ptr()
    job.desc = ctypes.pointer(plan.desc)
    job.out_offset = out_offset
    job.store_kind = store_kind
    job.tile_elements = info["tile_elements"]
    job.rows, job.cols_padded = info["rows"], info["cols"]
    job.error_dev = plan.error.data_ptr()
    return job


#: Activation rows the multiply-on-the-fly kernels take at most, and the shortest weight row they handle.
FUSED_MAX_ROWS = 4
FUSED_MIN_COLS = 256


def fused_linear_usable(buffers: LatticeBuffers, shape, x: torch.Tensor) -> bool:
    """Can `linear_rows` take this container and activation? (Otherwise: decode, then multiply.)"""
    rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
    return (x.dtype == torch.bfloat16 and 0 < rows <= FUSED_MAX_ROWS and shape[1] % 8 == 0 and shape[1] >= FUSED_MIN_COLS
            and x.shape[-1] == shape[1] and buffers.payload.device.type == "cuda")


def fused_linear_pays(buffers: LatticeBuffers, shape, x: torch.Tensor) -> bool:
    """Usable, and measured faster than decoding and multiplying separately.

    One row always pays (8192 x 28672 @ 4 bpp: 175 us against 233 us; on a 3072 x 3072 weight the two are level and
    this one never writes the weight). Two to four rows pay on weights whose decode is bound by throughput (more tile
    pairs than 16 waves on every CU hold): the extra products ride along in issue slots the decode leaves free
    (8192 x 28672: 217 us against 224 us at 4 bpp, 275 against 290 at 8 bpp). On a smaller weight the launch lasts as
    long as one tile's chain of dependent steps, the products lengthen every link of it, and decoding first is faster
    (3072 x 3072, four rows: 103 us against 84 us).
    """
    if not fused_linear_usable(buffers, shape, x):
        return False
    info, _, _ = _checked_geometry(buffers, shape, torch.bfloat16)
    with torch.cuda.device(buffers.payload.device):
        plan = _plan_for(buffers, info)
    if plan.desc.table_kind == _hip.TABLE_GLOBAL64:
        return False
    rows = x.numel() // x.shape[-1]
    if rows == 1:
        return True
    device = buffers.payload.device
    caps = _hip.device_info(device.index if device.index is not None else torch.cuda.current_device())
    pairs = (int(buffers.states.shape[0]) + 1) // 2
    return pairs > 16 * caps.compute_units


def linear_rows(buffers: LatticeBuffers, *, shape, x: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
    """x[..., K] @ W.T (+ bias) for up to four activation rows, W = this bf16 container, without ever writing W.

    ep_hip_linear_fused_bf16: the decode kernel multiplies each decoded vector with the activations in registers.
    The reference decodes the whole weight and calls F.linear (entropack/linear/linear.py:163-165).
    """
    device = buffers.payload.device
    info, out_dtype, _ = _checked_geometry(buffers, shape, torch.bfloat16)
    if not fused_linear_usable(buffers, shape, x):
        raise ValueError("linear_rows takes 1..4 bfloat16 activation rows and weight rows of a multiple of 8, at least 256, columns")
    flat = x.reshape(-1, x.shape[-1])
    if flat.stride(-1) != 1 or flat.stride(0) % 8 or flat.data_ptr() % 16:
        flat = flat.contiguous()
    outer = info["rows"]
    with torch.cuda.device(device):
        plan = _plan_for(buffers, info)
        job = _job_of(buffers, info, plan, _hip.STORE_KINDS[torch.bfloat16])
        out = torch.empty(flat.shape[0], outer, dtype=x.dtype, device=device)
        workspace = torch.empty(flat.shape[0] * outer, dtype=torch.float32, device=device)
        bias_ready = None if bias is None else bias.to(device=device, dtype=x.dtype).contiguous()
        _hip.check("ep_hip_linear_fused_bf16", _hip.library().ep_hip_linear_fused_bf16(
            ctypes.byref(job), flat.data_ptr(), flat.shape[0], flat.stride(0), None if bias_ready is None else bias_ready.data_ptr(),
            out.data_ptr(), out.stride(0), _hip.FLOAT_KINDS[x.dtype], workspace.data_ptr(), _hip.current_stream(device)))
    return out.reshape(*x.shape[:-1], outer)


def fused_batches(buffers: LatticeBuffers, info: dict) -> tuple[torch.Tensor, int, int]:
    """(device table of ep_hip_fused_batch, number of batches, number of tiles) for decode-to-GEMM through LDS, built once
    per container and kept on its `layout` tensor: ep_hip_fused_plan groups the tiles whose chains stay aligned in k."""
    device = buffers.payload.device
    key = (info["rows"], info["cols"], info["tile_elements"], device)
    cached = getattr(buffers.layout, "_lattice_rans_hip_fused_batches", None)
    if cached is not None and cached[0] == key:
        return cached[1:]
    lib = _hip.library()
    count = ctypes.c_int(0)
    _hip.check("ep_hip_fused_plan", lib.ep_hip_fused_plan(info["rows"], info["cols"], info["tile_elements"], None, 0, ctypes.byref(count)))
    host = torch.zeros(count.value * ctypes.sizeof(_hip.FusedBatch), dtype=torch.uint8)
    _hip.check("ep_hip_fused_plan", lib.ep_hip_fused_plan(info["rows"], info["cols"], info["tile_elements"], host.data_ptr(), count.value,
                                                          ctypes.byref(count)))
    table = host.to(device)
    buffers.layout._lattice_rans_hip_fused_batches = (key, table, count.value, info["total_tiles"])
    return table, count.value, info["total_tiles"]


def mfma_linear_usable(buffers: LatticeBuffers, shape, x: torch.Tensor) -> bool:
    """Can `linear_mfma` (bfloat16 activations) or `linear_mfma_i8` (int8 activation codes) take this container and
    activation? Weight rows of a multiple of 32 and at least 256 columns, and a plan with the two-level tables of prob_bits
    11 (what the default encoder settings give up to 7 bpp)."""
    if not (x.dtype in (torch.bfloat16, torch.int8) and x.numel() > 0 and shape[1] % 32 == 0 and shape[1] >= 256 and x.shape[-1] == shape[1]
            and buffers.payload.device.type == "cuda"):
        return False
    info, _, _ = _checked_geometry(buffers, shape, x.dtype)
    with torch.cuda.device(buffers.payload.device):
        plan = _plan_for(buffers, info)
    return plan.desc.prob_bits == 11 and plan.desc.sym_offset != 0 and plan.desc.table_kind in (_hip.TABLE_LDS_BYTE, _hip.TABLE_LDS_SYM)


def _mfma_call(buffers: LatticeBuffers, shape, flat: torch.Tensor, weight_dtype: torch.dtype, out_dtype: torch.dtype, bias, extra):
    """Common part of the two decode-to-GEMM calls: plan, batches, job, output, workspace; `extra(job, table, batches, out,
    workspace, bias pointer, stream)` makes the C call."""
    device = buffers.payload.device
    info, _, _ = _checked_geometry(buffers, shape, weight_dtype)
    if not mfma_linear_usable(buffers, shape, flat):
        raise ValueError("decode-to-GEMM through LDS takes bfloat16 or int8 activations, weight rows of a multiple of 32 (at least 256) "
                         "columns and a container whose plan has the two-level tables (prob_bits 11, byte-valued symbols)")
    outer = info["rows"]
    with torch.cuda.device(device):
        plan = _plan_for(buffers, info)
        table, batches, _ = fused_batches(buffers, info)
        job = _job_of(buffers, info, plan, _hip.STORE_KINDS[weight_dtype])
        out = torch.empty(flat.shape[0], outer, dtype=out_dtype, device=device)
        workspace = torch.empty(_hip.library().ep_hip_linear_fused_mfma_workspace(outer, info["cols"], info["tile_elements"], flat.shape[0],
                                                                                   1 if weight_dtype == torch.int8 else 0),
                                dtype=torch.uint8, device=device)
        bias_ready = None if bias is None else bias.to(device=device, dtype=out_dtype).contiguous()
        extra(job, table, batches, out, workspace, None if bias_ready is None else bias_ready.data_ptr(), _hip.current_stream(device))
    return out


def linear_mfma(buffers: LatticeBuffers, *, shape, x: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
    """x[..., K] @ W.T (+ bias) for any number of activation rows, W = this bf16 container, the decoded weight going from the
    rANS lanes to the matrix cores through LDS and never to memory (ep_hip_linear_fused_mfma_bf16).

    The reference decodes the whole weight and calls F.linear (entropack/linear/linear.py:163-165).
    """
    flat = x.reshape(-1, x.shape[-1])
    if flat.stride(-1) != 1 or flat.stride(0) % 8 or flat.data_ptr() % 16:
        flat = flat.contiguous()

    def call(job, table, batches, out, workspace, bias_pointer, stream):
        _hip.check("ep_hip_linear_fused_mfma_bf16", _hip.library().ep_hip_linear_fused_mfma_bf16(
            ctypes.byref(job), table.data_ptr(), batches, flat.data_ptr(), flat.shape[0], flat.stride(0), bias_pointer, out.data_ptr(),
            out.stride(0), _hip.FLOAT_KINDS[x.dtype], workspace.data_ptr(), stream))

    out = _mfma_call(buffers, shape, flat, torch.bfloat16, x.dtype, bias, call)
    return out.reshape(*x.shape[:-1], out.shape[-1])


def linear_mfma_i8(buffers: LatticeBuffers, *, shape, activation: torch.Tensor, activation_scale: torch.Tensor, weight_scale: torch.Tensor,
                   bias: torch.Tensor | None, out_dtype: torch.dtype) -> torch.Tensor:
    """W8A8 with the int8 weight codes decoded inside the product (ep_hip_linear_fused_mfma_i8): `activation` int8 [M, K] with
    `activation_scale` f32[M] (ep_hip_quantize_rows), `weight_scale` f32[N]; the same bits as the int8 GEMM on decoded codes.

    The reference decodes the codes and calls its Triton int8 GEMM (entropack/linear/linear.py:362-385,485-490).
    """
    flat = activation.reshape(-1, activation.shape[-1])
    if flat.stride(-1) != 1 or flat.stride(0) % 16 or flat.data_ptr() % 16:
        flat = flat.contiguous()
    scale_a = activation_scale.to(device=flat.device, dtype=torch.float32).contiguous()
    scale_b = weight_scale.to(device=flat.device, dtype=torch.float32).contiguous()

    def call(job, table, batches, out, workspace, bias_pointer, stream):
        _hip.check("ep_hip_linear_fused_mfma_i8", _hip.library().ep_hip_linear_fused_mfma_i8(
            ctypes.byref(job), table.data_ptr(), batches, flat.data_ptr(), flat.shape[0], flat.stride(0), scale_a.data_ptr(), scale_b.data_ptr(),
            bias_pointer, out.data_ptr(), out.stride(0), _hip.FLOAT_KINDS[out_dtype], workspace.data_ptr(), stream))

    return _mfma_call(buffers, shape, flat, torch.int8, out_dtype, bias, call)


class BatchDecoder:
    """Decodes many containers (a model's layers) in one pass: ep_hip_batch_plan / ep_hip_decode_lattice_batch.

    Containers that share a kernel variant go into one launch whose workgroups each take a slice of one container, so
    layers too small to fill the device on their own run side by side. The plan (argument blocks and the block map)
    is built once and reused for every pass, like the per-container plans it refers to. The reference decodes layer
    by layer (entropack/linear/linear.py:125-130 called from each module's forward) and has no batched entry.
    """

    def __init__(self, items):
        """items: iterable of (LatticeBuffers, shape, dtype); all on one device."""
        items = list(items)
        if not items:
            raise ValueError("BatchDecoder needs at least one container")
        self.device = items[0][0].payload.device
        self._keep = []                       # plans, descs and buffers the device-side argument blocks point into
        self._views = []                      # (byte offset, rows, cols, out dtype, final dtype or None)
        jobs = (_hip.DecodeJob * len(items))()
        cursor = 0
        with torch.cuda.device(self.device):
            for job, (buffers, shape, dtype) in zip(jobs, items):
                if buffers.payload.device != self.device:
                    raise ValueError("every container of a batch must live on the same device")
                info, out_dtype, via_float32 = _checked_geometry(buffers, shape, dtype)
                plan = _plan_for(buffers, info)
                rows, cols = info["rows"], info["cols"]
                filled = _job_of(buffers, info, plan, _hip.STORE_KINDS[out_dtype], cursor)
                ctypes.memmove(ctypes.byref(job), ctypes.byref(filled), ctypes.sizeof(_hip.DecodeJob))
                self._keep.append((plan, buffers))
                self._views.append((cursor, rows, cols, out_dtype, dtype if via_float32 else None))
                cursor += -(-rows * cols * out_dtype.itemsize // 256) * 256
            self.arena_bytes = cursor
            lib = _hip.library()
            caps = _hip.device_info(self.device.index if self.device.index is not None else torch.cuda.current_device())
            size = ctypes.c_size_t(0)
            _hip.check("ep_hip_batch_plan", lib.ep_hip_batch_plan(jobs, len(items), caps.compute_units, None, ctypes.byref(size)))
            self._blob_host = torch.zeros(size.value, dtype=torch.uint8)
            _hip.check("ep_hip_batch_plan", lib.ep_hip_batch_plan(
                jobs, len(items), caps.compute_units, self._blob_host.data_ptr(), ctypes.byref(size)))
            self._blob_dev = self._blob_host.to(self.device)

    def decode(self, arena: torch.Tensor | None = None) -> list[torch.Tensor]:
        """One pass over every container on torch's current stream; returns `[rows, padded cols]` views of the arena.

        `arena` (uint8, at least `arena_bytes`, 256-byte aligned) lets a caller reuse one output buffer pass after pass.
        """
        with torch.cuda.device(self.device):
            if arena is None:
                arena = torch.empty(self.arena_bytes, dtype=torch.uint8, device=self.device)
            elif arena.device != self.device or arena.dtype != torch.uint8 or arena.numel() < self.arena_bytes \
                    or not arena.is_contiguous() or arena.data_ptr() % 256:
                raise ValueError("arena must be a contiguous, 256-byte aligned uint8 tensor of at least arena_bytes on the batch's device")
            _hip.check("ep_hip_decode_lattice_batch", _hip.library().ep_hip_decode_lattice_batch(
                self._blob_host.data_ptr(), self._blob_dev.data_ptr(), arena.data_ptr(), _hip.current_stream(self.device)))
        outputs = []
        for offset, rows, cols, out_dtype, final in self._views:
            view = arena[offset:offset + rows * cols * out_dtype.itemsize].view(out_dtype).view(rows, cols)
            outputs.append(snap_to_container(view, final) if final is not None else view)
        return outputs

    def check_errors(self) -> None:
        for _, buffers in self._keep:
            check_errors(buffers)


def launch_table_kind(buffers: LatticeBuffers, *, shape, dtype) -> str:
    """Name of the table form a decode of this container to `dtype` runs with (after at least one decode)."""
    plan = plan_of(buffers)
    if plan is None:
        raise RuntimeError("the container has not been decoded yet")
    info, out_dtype, _ = _checked_geometry(buffers, shape, dtype)
    device = buffers.payload.device
    caps = _hip.device_info(device.index if device.index is not None else torch.cuda.current_device())
    kind = _hip.library().ep_hip_decode_table_kind(ctypes.byref(plan.desc), _hip.STORE_KINDS[out_dtype], info["rows"], info["cols"],
                                                   info["tile_elements"], caps.compute_units)
    return _hip.TABLE_KIND_NAMES[kind]


def plan_of(buffers: LatticeBuffers) -> DecodePlan | None:
    """The cached plan of a container that has been decoded at least once."""
    return getattr(buffers.layout, "_lattice_rans_hip_plan", None)


def check_errors(buffers: LatticeBuffers) -> None:
    """Synchronises and raises ValueError if any decode of this container flagged a corrupt stream.

    The reference passes an error word to its kernels and never reads it (cuda.py:756,765,773); here it can be read
    on demand, off the hot path.
    """
    plan = plan_of(buffers)
    if plan is None:
        return
    code = int(plan.error.item())
    if code:
        plan.error.zero_()
        raise ValueError(f"lattice_rans decode error {code}: {_hip.DECODE_ERRORS.get(code, 'unknown')}")


def encode(**kwargs):
    """Lane contract of the reference's CUDA lane (entropack/schemes/lattice_rans/cuda.py:561-597): the weight is on the
    device and so are the buffers returned. The kernels and their orchestration live in hip_encode.py."""
    from . import hip_encode
    return hip_encode.encode(**kwargs)
