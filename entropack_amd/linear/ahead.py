"""Decoding the weights of a layer sequence a group at a time, ahead of their use.

A single weight of a few million parameters cannot fill the GPU: a tile is one long chain of dependent rANS steps, so
the decode of one 3072 x 3072 layer lasts as long as one tile's chain (about 85 us) whatever the bandwidth, which is
more than the layer's whole product at 4096 activation rows. `DecodeAhead` takes the compressed layers of a model in
the order they run, decodes `group_size` of them per pass (one launch set, every tile of the group side by side: the
launch is then bound by bandwidth, not by one chain) into an arena, and hands each layer its dense weight as a view
when the layer's forward asks for it. By default the pass runs on the layers' own stream, between the products of
two groups, and one group of dense weights is held. With `overlap=True` it runs on a second stream into one of two
arenas while the previous group multiplies. On an MI355X the first is the faster one for 3072 x 3072 layers at 4096
activation rows (71 against 73 us per layer in bf16, 63 against 65 us in W8A8): a decode that runs beside the
products takes compute units and bandwidth from them, and costs them more than the 8 us per layer it needs alone.

The reference decodes every layer inside its own forward (entropack/linear/linear.py:125-130,163-165); it has no
counterpart of this class.
"""
from __future__ import annotations

import torch

from ..compression import BatchDecompressor, CompressedTensor


class DecodeAhead:
    """Attach to `layers` (compressed linear layers with `lattice_rans` weights on one GPU, in execution order).

    Forward passes then take their weights from here whenever autograd does not need to keep them; a layer asked for
    out of order is served too (its group is decoded on the spot), so correctness never depends on the order, only
    the overlap does. `close()` detaches. Not thread-safe: one forward pass at a time.
    """

    def __init__(self, layers, group_size: int = 8, overlap: bool = False):
        self._layers = list(layers)
        if not self._layers:
            raise ValueError("DecodeAhead needs at least one layer")
        if isinstance(group_size, bool) or not isinstance(group_size, int) or group_size < 1:
            raise ValueError(f"group_size must be a positive integer, got {group_size!r}")
        devices = set()
        for layer in self._layers:
            weight = getattr(layer, "weight", None)
            if not isinstance(weight, CompressedTensor) or weight.compress_method != "lattice_rans":
                raise ValueError(f"DecodeAhead takes layers whose weight is a lattice_rans container, got {type(layer).__name__} "
                                 f"with {type(weight).__name__}")
            if getattr(layer, "_decode_ahead", None) is not None:
                raise ValueError("a layer is already attached to another DecodeAhead")
            devices.add(weight.device)
        if len(devices) != 1 or next(iter(devices)).type != "cuda":
            raise ValueError(f"all layers must hold their weights on one GPU, got {sorted(str(d) for d in devices)}")
        self.device = next(iter(devices))
        self.group_size = group_size
        self.overlap = bool(overlap)
        self._index = {id(layer): position for position, layer in enumerate(self._layers)}
        if len(self._index) != len(self._layers):
            raise ValueError("a layer appears twice in the sequence")
        config = self._layers[0]._decode_config
        self._groups = [self._layers[first:first + group_size] for first in range(0, len(self._layers), group_size)]
        with torch.cuda.device(self.device):
            self._decoders = [BatchDecompressor([layer.weight for layer in group], config) for group in self._groups]
            room = max(decoder.arena_bytes for decoder in self._decoders)
            self._arenas = [torch.empty(room, dtype=torch.uint8, device=self.device) for _ in range(min(2, len(self._groups)) if self.overlap else 1)]
            self._side = torch.cuda.Stream(device=self.device) if self.overlap else None
        self._slots = [None] * len(self._arenas)        # per arena: (group, [dense weights], ready event)
        self._recent = len(self._arenas) - 1             # the arena served last
        for layer in self._layers:
            layer._decode_ahead = self

    @property
    def arena_bytes(self) -> int:
        """Dense bytes held for as long as this object lives."""
        return sum(arena.numel() for arena in self._arenas)

    def close(self) -> None:
        """Detach from the layers. Work already queued keeps its weights: the arenas are not reused before it ran."""
        for layer in self._layers:
            if getattr(layer, "_decode_ahead", None) is self:
                layer._decode_ahead = None
        if self._side is not None:
            with torch.cuda.device(self.device):
                torch.cuda.current_stream(self.device).wait_stream(self._side)     # a decode nobody took may still be writing
        self._slots = [None] * len(self._arenas)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- decoding ---------------------------------------------------------------------------------------------------

    def _slot_of(self, group: int):
        for slot, held in enumerate(self._slots):
            if held is not None and held[0] == group:
                return slot
        return None

    def _start(self, group: int, slot: int, user: torch.cuda.Stream) -> None:
        """Decode `group` into arena `slot`. Whatever `user` has queued so far may still read that arena: wait for it."""
        if self._side is None:
            self._slots[slot] = (group, self._decoders[group](self._arenas[slot]), None)
            return
        released = torch.cuda.Event()
        released.record(user)
        self._side.wait_event(released)
        with torch.cuda.stream(self._side):
            dense = self._decoders[group](self._arenas[slot])
            ready = torch.cuda.Event()
            ready.record(self._side)
        self._slots[slot] = (group, dense, ready)

    def weight_of(self, layer) -> torch.Tensor | None:
        """The dense weight (container dtype) of an attached layer, a view of an arena: valid for the work queued before
        the first layer of the next group but one asks for its weight. None for a layer that is not attached here."""
        position = self._index.get(id(layer))
        if position is None:
            return None
        group, offset = divmod(position, self.group_size)
        with torch.cuda.device(self.device):
            user = torch.cuda.current_stream(self.device)
            slot = self._slot_of(group)
            if slot is None:                                   # first pass, or a layer out of sequence
                slot = (self._recent + 1) % len(self._arenas)
                self._start(group, slot, user)
            self._recent = slot
            held = self._slots[slot]
            if held[2] is not None:
                user.wait_event(held[2])
            # The first layer of a group starts the next group's decode, which then runs beside this group's products.
            if len(self._arenas) > 1 and offset == 0:
                following = (group + 1) % len(self._groups)
                if self._slot_of(following) is None:
                    self._start(following, 1 - slot, user)
        return held[1][offset]

    def check_errors(self) -> None:
        for decoder in self._decoders:
            decoder.check_errors()
