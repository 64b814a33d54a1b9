"""Per-block decompress(-ahead) for a converted model.

The reference decompresses a weight inside the very call that needs it, one
tensor per kernel sequence, and blocks the host until it is there
(cuda/high_level.cu:203,252-263).  A single projection matrix is too small to
fill an MI355X with decoder wavefronts, the seven of a transformer block
together are not.  ``DecompressAhead`` therefore decodes all compressed Linear
weights of one block with ONE kernel launch into a static dense buffer, at the
moment the block's first Linear runs, and (``ahead=True``) already enqueues
the next block's decode on a side stream so that it overlaps the current
block's GEMMs.  Only HIP streams and events are used; all streams have the
default priority; nothing is allocated after construction.

Usage::

    manager.convert(model); model.cuda()
    ahead = DecompressAhead(manager, model)      # blocks = elements of the model's ModuleLists
    with ahead:                                   # or ahead.enable() / ahead.disable()
        y = model(x)
"""
from __future__ import annotations

import torch

from neuzip_amd.nn.linear import Linear


def _default_blocks(model: torch.nn.Module):
    """Elements of every ModuleList that hold compressed Linears, in module order."""
    blocks = []
    for mod in model.modules():
        if isinstance(mod, torch.nn.ModuleList):
            for child in mod:
                if any(isinstance(m, Linear) for m in child.modules()):
                    blocks.append(child)
    # a nested ModuleList would list a Linear twice: keep the outermost grouping
    seen, out = set(), []
    for b in blocks:
        lins = [m for m in b.modules() if isinstance(m, Linear) and id(m) not in seen]
        if lins:
            seen.update(id(m) for m in lins)
            out.append(lins)
    return out


class _Slot:
    """One static dense buffer able to hold the weights of any block."""

    __slots__ = ("buf", "ready", "block", "stamps")

    def __init__(self, numel: int, device):
        self.buf = torch.empty(numel, dtype=torch.bfloat16, device=device)
        self.ready = None  # event of a side-stream decode the consumer has not waited for yet
        self.block = -1    # index of the block whose weights the buffer holds (or will hold)
        self.stamps = []   # per tensor of that block: the handle's write count when it was decoded


_MAX_TENSORS = 16  # tensors one decode launch takes (NZ_BATCH_MAX)


def _merge_small(groups, numel, fill: int):
    """Consecutive blocks whose weights are too few to fill the device share a
    launch: blocks are added to a group until it holds ``fill`` elements (or 16
    tensors).  A launch takes as long as its longest segment however few of them
    there are, so the four weights of a GPT-2-medium block (12.6 M elements, 92
    chunks on 256 compute units) cost as much alone as three such blocks together."""
    out = []
    for g in groups:
        if out and len(out[-1]) + len(g) <= _MAX_TENSORS and sum(numel(m) for m in out[-1]) < fill:
            out[-1] = out[-1] + g
        else:
            out.append(list(g))
    return out


class DecompressAhead:
    def __init__(self, manager, model: torch.nn.Module, blocks=None, ahead: bool = True, wrap: bool = True,
                 merge_small: bool = True):
        """``blocks``: modules whose compressed Linears are decoded together
        (default: the elements of the model's ModuleLists, small ones merged
        until a launch gives every SIMD unit of the device two wavefronts,
        unless ``merge_small`` is off); ``ahead``: decode block k+1 on a side
        stream while block k computes; ``wrap``: after the last block, already
        decode the first one for the next forward pass."""
        self.manager = manager
        self.wrap = bool(wrap)
        be = manager._be
        groups = _default_blocks(model) if blocks is None else [
            [m for m in b.modules() if isinstance(m, Linear)] for b in blocks]
        if blocks is None and merge_small:
            cus = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
            groups = _merge_small([g for g in groups if g], lambda m: be.numel(m._p._handle), 2 * 4 * cus * 64 * 256)
        self._handles = [[m._p._handle for m in g] for g in groups if g]
        self._where = {}
        for bi, hs in enumerate(self._handles):
            for k, h in enumerate(hs):
                self._where[h] = (bi, k)
        self.tensors_per_launch = [len(hs) for hs in self._handles]
        self._plans = [be.batch_plan(hs) for hs in self._handles]
        self._single = {}  # (block, k) -> plan that decodes that one tensor again after a write
        # element offsets of the block's tensors in a slot buffer, 16-byte aligned
        self._offsets, need = [], 0
        for hs in self._handles:
            offs, at = [], 0
            for h in hs:
                offs.append(at)
                at += (be.numel(h) + 7) & ~7
            self._offsets.append(offs)
            need = max(need, at)
        dev = torch.device("cuda", torch.cuda.current_device())
        self.ahead = bool(ahead) and len(self._handles) > 1
        self._slots = [_Slot(need, dev) for _ in range(2 if self.ahead else 1)]
        self._views = [[[s.buf[o:o + be.numel(h)] for o, h in zip(offs, hs)]
                        for offs, hs in zip(self._offsets, self._handles)] for s in self._slots]
        self.stream = torch.cuda.Stream() if self.ahead else None  # default priority
        self._enabled = False
        self._last, self._step = -1, 1  # block visited last, direction of the walk

    # -- context management ---------------------------------------------------
    def enable(self):
        if not self._enabled:
            self.manager.linear = self._linear  # instance attributes shadow the methods
            self.manager.read_shared = self._read_shared
            self.manager._on_write = self._before_write
            self._enabled = True

    def disable(self):
        if self._enabled:
            del self.manager.linear
            del self.manager.read_shared
            self.manager._on_write = None
            self.join()
            self._enabled = False

    def __enter__(self):
        self.enable()
        return self

    def __exit__(self, *exc):
        self.disable()
        return False

    def join(self):
        """Make the current stream wait for any decode still running on the side
        stream and forget what the buffers hold (call before ending a stream
        capture).  Writes through the manager need no call: a decoded tensor is
        used only while its handle's write count is what it was at decode time,
        and only that tensor is decoded again."""
        cur = torch.cuda.current_stream()
        for s in self._slots:
            if s.ready is not None:
                cur.wait_event(s.ready)
            s.ready = None
            s.block = -1
            s.stamps = []
        self._last, self._step = -1, 1

    # -- the hook ---------------------------------------------------------------
    # Stream order does most of the work: the consumer stream decodes, computes
    # and releases buffers in program order; the side stream is forked from the
    # consumer stream at the entry of a block (one event) and joined at the
    # entry of the next one (one event).
    def _decode_here(self, bi: int, slot_i: int, cur) -> None:
        slot = self._slots[slot_i]
        if slot.ready is not None:  # an unused decode-ahead still owns the buffer
            cur.wait_event(slot.ready)
            slot.ready = None
        self.manager._be.read_batch(self._plans[bi], self._views[slot_i][bi])
        slot.block = bi
        slot.stamps = self._stamps_now(bi)

    def _decode_ahead(self, bi: int, slot_i: int, cur) -> None:
        slot = self._slots[slot_i]
        fork = torch.cuda.Event()
        fork.record(cur)  # every earlier reader and writer of the buffer is before this point
        with torch.cuda.stream(self.stream):
            self.stream.wait_event(fork)
            self.manager._be.read_batch(self._plans[bi], self._views[slot_i][bi])
            slot.ready = torch.cuda.Event()
            slot.ready.record(self.stream)
        slot.block = bi
        slot.stamps = self._stamps_now(bi)

    def _stamps_now(self, bi: int):
        stamps = self.manager._stamps
        return [stamps.get(h, 0) for h in self._handles[bi]]

    def _before_write(self, handle: str) -> None:
        """A write may encode in place, over the container a decode-ahead on the
        side stream is still reading: the writing stream waits for that decode."""
        where = self._where.get(handle)
        if where is None:
            return
        for s in self._slots:
            if s.block == where[0] and s.ready is not None:
                torch.cuda.current_stream().wait_event(s.ready)

    def _weight(self, handle: str):
        bi, k = self._where[handle]
        slot_i = next((i for i, s in enumerate(self._slots) if s.block == bi), None)
        entering = bi != self._last
        if entering:
            # backward passes walk the blocks in reverse; the step from the last block
            # to the first one is the start of the next forward pass
            self._step = -1 if bi == self._last - 1 else 1
            self._last = bi
        cur = torch.cuda.current_stream()
        if entering or slot_i is None:
            if slot_i is None:
                slot_i = next((i for i, s in enumerate(self._slots) if s.block < 0), 0)
                self._decode_here(bi, slot_i, cur)
            slot = self._slots[slot_i]
            if slot.ready is not None:  # join the side stream once per block
                cur.wait_event(slot.ready)
                slot.ready = None
            nxt = bi + self._step
            if self.ahead and entering and (self.wrap or 0 <= nxt < len(self._handles)):
                nxt %= len(self._handles)
                other = 1 - slot_i
                if self._slots[other].block != nxt:
                    if self._slots[other].ready is not None:  # never consumed: keep the streams joined
                        cur.wait_event(self._slots[other].ready)
                        self._slots[other].ready = None
                    self._decode_ahead(nxt, other, cur)
        elif self._slots[slot_i].ready is not None:
            cur.wait_event(self._slots[slot_i].ready)
            self._slots[slot_i].ready = None
        slot = self._slots[slot_i]
        now = self.manager._stamps.get(handle, 0)
        if slot.stamps[k] != now:  # written since the block was decoded: this tensor again, the others stay
            plan = self._single.get((bi, k))
            if plan is None:
                plan = self._single[(bi, k)] = self.manager._be.batch_plan([handle])
            self.manager._be.read_batch(plan, [self._views[slot_i][bi][k]])
            slot.stamps[k] = now
        return self._views[slot_i][bi][k]

    def _read_shared(self, handle: str) -> torch.Tensor:
        if handle in self._where:
            return self._weight(handle).view(self.manager.meta_dict[handle])
        return type(self.manager).read_shared(self.manager, handle)

    def _linear(self, handle: str, inputs: torch.Tensor, bias=None) -> torch.Tensor:
        shape = self.manager.meta_dict[handle]
        if handle in self._where:
            weight = self._weight(handle)
        else:
            weight = self.manager._be.read(handle)
        weight = weight.view(shape)
        if bias is not None and inputs.dim() == 2:
            return torch.addmm(bias, inputs, weight.t())
        return torch.nn.functional.linear(inputs, weight, bias)
