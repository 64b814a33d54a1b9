"""Decompress-ahead for a converted model.

The reference decompresses a weight inside the very call that needs it and
blocks the host until it is there (cuda/high_level.cu:203,252-263).  Here the
weight of the NEXT compressed Linear is decoded on a side stream while the
current one runs its GEMM, so that by the time a layer is reached its dense
weight is (partly) ready.  Only HIP streams and events are used; all streams
have the default priority.

Usage::

    manager.convert(model); model.cuda()
    ahead = DecompressAhead(manager, model)      # forward order = module order
    with ahead:                                   # or ahead.enable() / ahead.disable()
        y = model(x)
"""
from __future__ import annotations

import torch

from neuzip_amd.nn.linear import Linear


class _Slot:
    """One dense scratch buffer of the ring kept per weight size."""

    __slots__ = ("buf", "ready", "free", "handle")

    def __init__(self, numel: int, device):
        self.buf = torch.empty(numel, dtype=torch.bfloat16, device=device)
        self.ready = None   # recorded on the side stream when the decode is enqueued
        self.free = None    # recorded on the consumer's stream after the GEMM that used the buffer
        self.handle = None


class DecompressAhead:
    def __init__(self, manager, model: torch.nn.Module, depth: int = 1):
        self.manager = manager
        self.layers = [m for m in model.modules() if isinstance(m, Linear)]
        self.handles = [m._p._handle for m in self.layers]
        self.depth = max(1, int(depth))
        self.stream = torch.cuda.Stream()  # default priority
        self._pos = {h: i for i, h in enumerate(self.handles)}
        be = manager._be
        self._numel = {h: be.numel(h) for h in self.handles}
        # a ring of depth + 1 dense buffers per distinct weight size: one being
        # consumed, `depth` being filled
        dev = torch.device("cuda", torch.cuda.current_device())
        self._rings = {}
        for n in set(self._numel.values()):
            self._rings[n] = [[_Slot(n, dev) for _ in range(self.depth + 1)], 0]
        self._ready = {}  # handle -> slot holding (or about to hold) its dense weight
        self._enabled = False

    # -- context management ---------------------------------------------------
    def enable(self):
        if not self._enabled:
            self.manager.linear = self._linear  # instance attribute shadows the method
            self._enabled = True

    def disable(self):
        if self._enabled:
            del self.manager.linear
            torch.cuda.synchronize()
            self._ready.clear()
            self._enabled = False

    def __enter__(self):
        self.enable()
        return self

    def __exit__(self, *exc):
        self.disable()
        return False

    # -- the hook ---------------------------------------------------------------
    def _issue(self, handle: str, after: torch.cuda.Event) -> None:
        if handle in self._ready:
            return
        ring = self._rings[self._numel[handle]]
        slot = ring[0][ring[1]]
        ring[1] = (ring[1] + 1) % len(ring[0])
        if slot.handle is not None:
            self._ready.pop(slot.handle, None)  # evicted before use
        with torch.cuda.stream(self.stream):
            self.stream.wait_event(after)          # not further ahead than `depth` layers
            if slot.free is not None:
                self.stream.wait_event(slot.free)  # the last consumer of this buffer is done
            self.manager._be.read_into(handle, slot.buf)
            slot.ready = torch.cuda.Event()
            slot.ready.record(self.stream)
        slot.handle = handle
        self._ready[handle] = slot

    def _linear(self, handle: str, inputs: torch.Tensor, bias=None) -> torch.Tensor:
        shape = self.manager.meta_dict[handle]
        cur = torch.cuda.current_stream()
        i = self._pos.get(handle)
        slot = self._ready.pop(handle, None)
        if slot is None:
            weight = self.manager._be.read(handle)
        else:
            cur.wait_event(slot.ready)
            weight = slot.buf
            slot.handle = None
        if i is not None:
            here = torch.cuda.Event()
            here.record(cur)
            n = len(self.handles)
            for k in range(1, self.depth + 1):
                self._issue(self.handles[(i + k) % n], here)
        weight = weight.view(shape)
        if bias is not None and inputs.dim() == 2:
            out = torch.addmm(bias, inputs, weight.t())
        else:
            out = torch.nn.functional.linear(inputs, weight, bias)
        if slot is not None:
            slot.free = torch.cuda.Event()
            slot.free.record(cur)
        return out
