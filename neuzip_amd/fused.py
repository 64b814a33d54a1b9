"""Fused decompress + matrix-vector product for single-token inference.

The reference's ``Manager::linear`` decompresses the weight into a dense
tensor and then calls ``addmm`` / ``matmul`` (cuda/high_level.cu:252-263).
For ONE activation row that doubles the memory traffic of the layer: the dense
weight is written once and read once, while the product itself needs every
weight exactly once.  ``FusedGemv`` routes such calls to a kernel that
multiplies while it decodes, and serves all Linears that consume the same
activation (q/k/v, gate/up) with one launch.  Calls with more than one row
keep the decompress-then-GEMM path.

Usage::

    fused = FusedGemv(manager, model)
    fused.trace(lambda: model(one_token))   # learns which Linears share their input
    with fused:
        y = model(one_token)

The result is deterministic (fixed summation order inside a wavefront, integer
accumulation across wavefronts) but not bit-identical to a GEMM library's.
"""
from __future__ import annotations

import ctypes

import torch

from neuzip_amd.nn.linear import Linear

_MAX_GROUP = 16


class _Group:
    __slots__ = ("handles", "names", "rows", "biases", "key", "outs", "in_features")

    def __init__(self, handles, rows, biases, in_features):
        self.handles = handles
        self.names = (ctypes.c_char_p * len(handles))(*[h.encode() for h in handles])
        self.rows = rows
        self.biases = biases
        self.in_features = in_features
        self.key = None
        self.outs = None


class FusedGemv:
    def __init__(self, manager, model: torch.nn.Module):
        self.manager = manager
        self._layers = {m._p._handle: m for m in model.modules() if isinstance(m, Linear)}
        self._groups = []
        self._where = {}
        self._enabled = False
        self._recording = None
        for h, m in self._layers.items():  # until traced: every Linear on its own
            self._add_group([h])

    # -- grouping -----------------------------------------------------------------
    def _eligible(self, handle) -> bool:
        m = self._layers.get(handle)
        return m is not None and m.in_features % 512 == 0 and m._p.dtype == torch.bfloat16

    def _add_group(self, handles):
        if not all(self._eligible(h) for h in handles):
            return
        mods = [self._layers[h] for h in handles]
        g = _Group(list(handles), [m.out_features for m in mods], [m.bias for m in mods], mods[0].in_features)
        self._groups.append(g)
        for k, h in enumerate(handles):
            self._where[h] = (g, k)

    def trace(self, fn, regroup: bool = True) -> None:
        """Run ``fn()`` once on the ordinary path and group the Linears that were
        called back to back with the very same single-row input tensor.  With a
        manager that chooses the geometry per tensor, the matrices of a group
        are then stored again with a geometry chosen for the group (``regroup``)."""
        self._recording = []
        was = self._enabled
        self.enable()
        try:
            with torch.no_grad():
                fn()
        finally:
            if not was:
                self.disable()
            rec, self._recording = self._recording, None
        self._groups, self._where = [], {}
        run, run_key = [], None
        for handle, key in rec + [(None, None)]:
            if run and (key is not run_key or key is None or len(run) == _MAX_GROUP or handle in run):
                self._add_group(run)
                run = []
            if handle is not None and key is not None:
                run.append(handle)
                run_key = key
        for h in self._layers:
            if h not in self._where:
                self._add_group([h])
        if regroup and getattr(self.manager._be, "auto_geometry", False):
            for g in self._groups:
                if len(g.handles) > 1:
                    self._fit_geometry(g)

    # Step time of a wavefront (ns) with one, two, three 8-wavefront workgroups per
    # compute unit, measured on MI355X; the same figures choose a tensor's geometry
    # when it is written on its own.
    _STEP_NS = (107, 147, 215)

    def _fit_geometry(self, g, cus=None) -> None:
        """Matrices that one launch decodes together are stored again with ONE
        geometry under which their chunks are a whole number of workgroups per
        compute unit (at most three, what a unit holds): chosen per tensor, two
        512-chunk matrices are a round of 768 workgroups and a poorly filled second.
        Only geometries inside the manager's size budget are considered; a group
        too small to fill the device with those keeps what it has."""
        be = self.manager._be
        if cus is None:
            cus = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
        sizes = [be.numel(h) for h in g.handles]
        best = None
        for k in (1, 2, 3):
            lane = -(-sum(sizes) // (k * cus * 512 * 8)) * 8
            while lane <= 512 and sum(-(-n // (lane * 512)) for n in sizes) > k * cus:
                lane += 8  # every tensor's last chunk is rounded up
            if not 64 <= lane <= 512 or not all(be.in_budget(n, lane * 512, lane) for n in sizes):
                continue
            t = lane * self._STEP_NS[k - 1]
            if best is None or t <= best[0]:  # measured on gate/up of an 8B model: 2 x 512 chunks 73-76 us, 2 x 256 71.5, 2 x 378 69.4
                best = (t, lane)
        if best is None:
            return
        lane = best[1]
        chunk = lane * 512
        if all(be.geometry(h) == (chunk, lane) for h in g.handles):
            return
        for h in g.handles:
            dense = self.manager.read(h)
            be.geometry_hint(h, chunk, lane)
            self.manager.write(dense, h)

    # -- context management ---------------------------------------------------
    def enable(self):
        if not self._enabled:
            self.manager.linear = self._linear  # instance attribute shadows the method
            self._enabled = True

    def disable(self):
        if self._enabled:
            del self.manager.linear
            self._enabled = False
            for g in self._groups:
                g.key = g.outs = None

    def __enter__(self):
        self.enable()
        return self

    def __exit__(self, *exc):
        self.disable()
        return False

    # -- the hook ---------------------------------------------------------------
    def _plain(self, handle, inputs, bias):
        return type(self.manager).linear(self.manager, handle, inputs, bias)

    def _linear(self, handle: str, inputs: torch.Tensor, bias=None) -> torch.Tensor:
        single_row = inputs.dim() >= 1 and inputs.numel() == inputs.shape[-1]
        if self._recording is not None:
            # the tensor object itself is the key (and is kept alive by the record, so
            # that neither its id nor its memory can be reused by a later activation)
            self._recording.append((handle, inputs if single_row else None))
            return self._plain(handle, inputs, bias)
        hit = self._where.get(handle)
        if (hit is None or not single_row or inputs.dtype != torch.bfloat16 or not inputs.is_cuda
                or inputs.shape[-1] != hit[0].in_features or torch.is_grad_enabled() and inputs.requires_grad):
            return self._plain(handle, inputs, bias)
        g, k = hit
        x = inputs if inputs.is_contiguous() else inputs.contiguous()
        key = (x.data_ptr(), x._version)
        if k == 0 or g.key != key or g.outs is None:
            if k != 0:  # called out of the traced order: this matrix alone
                out = torch.empty(g.rows[k], dtype=torch.bfloat16, device=x.device)
                names = (ctypes.c_char_p * 1)(g.names[k])
                self.manager._be.gemv_batch(names, x, [bias], [out])
                return out.view(*inputs.shape[:-1], g.rows[k])
            flat = torch.empty(sum(g.rows), dtype=torch.bfloat16, device=x.device)
            outs, at = [], 0
            for r in g.rows:
                outs.append(flat[at:at + r])
                at += r
            self.manager._be.gemv_batch(g.names, x, g.biases, outs)
            g.key, g.outs = key, outs
        out = g.outs[k]
        if k + 1 == len(g.handles):
            g.key = g.outs = None  # the group is served: do not keep the activation's identity alive
        if bias is not g.biases[k]:  # a bias other than the module's own: undo / apply by hand
            out = out.float()
            if g.biases[k] is not None:
                out = out - g.biases[k].float()
            if bias is not None:
                out = out + bias.float()
            out = out.to(torch.bfloat16)
        return out.view(*inputs.shape[:-1], g.rows[k])
