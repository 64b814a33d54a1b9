"""Python façade of the codec: ``Manager`` and ``Algorithm``.

Same surface as the reference's neuzip/binding.py:23-115 (constructor
arguments, method names, handle strings, return shapes); the backend is the
C ABI of libneuzip_hip.so instead of the pybind11 classes
``neuzip._cuda.Manager_f{precision}_n{normalizer_size}``.
"""
from __future__ import annotations

import ctypes
import enum
from typing import Optional

import torch

from neuzip_amd import _lib
from neuzip_amd._ahead import RequestOrder
from neuzip_amd.utils import _convert

_lib.load()  # hard failure when the extension is not built (reference: binding.py:15-20)


class Algorithm(enum.Enum):
    # neuzip/binding.py:23-27.  Only ANS has a native implementation here.
    ans = 0
    gdeflate = "gdeflate"
    zstd = "zstd"
    dummy = "dummy"


_VALID_NORMALIZERS = (0, 1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024)  # cuda/neuzip.cu:47-105


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class _AfterHeldWrites:
    """The library's functions as a manager's backend calls them: every
    ``nz_manager_*`` call first stores the writes the backend still holds back,
    so that no call can observe the store as it was before them."""

    def __init__(self, lib, owner):
        self._lib, self._owner, self._made = lib, owner, {}

    def __getattr__(self, name):
        fn = self._made.get(name)
        if fn is None:
            raw = getattr(self._lib, name)
            if name.startswith("nz_manager_"):
                owner = self._owner

                def fn(*args, _raw=raw):
                    if owner._held:
                        owner.flush()
                    return _raw(*args)
            else:
                fn = raw
            self._made[name] = fn
        return fn


class _HipBackend:
    """Backend object with the method set of the reference's C++ Manager
    (cuda/neuzip.cu:28-37): read / write / size / linear / linear_without_bias / split."""

    def __init__(self, precision: int, normalizer_size: int, chunk_size: int, lane_symbols: int,
                 size_budget: Optional[float] = None):
        self._raw = _lib.load()
        self._L = _AfterHeldWrites(self._raw, self)
        self._held = []  # writes held back: (handle, copy of the tensor, stream the copy was made on)
        self._held_elems = 0
        self.write_behind = True  # hold small writes back until 16 of them share a launch
        self._h = ctypes.c_void_p()
        self.auto_geometry = lane_symbols == "auto" and not chunk_size
        if lane_symbols == "auto":
            lane_symbols = _lib.LANE_SYMS_AUTO
        rc = self._L.nz_manager_create(_lib.ALGO_ANS, precision, normalizer_size, chunk_size,
                                       lane_symbols, ctypes.byref(self._h))
        _lib.raise_for(rc)
        if size_budget is not None:
            _lib.raise_for(self._L.nz_manager_set_size_budget(self._h, float(size_budget)))
        self._device = torch.device("cuda", torch.cuda.current_device())
        self._normalizer = int(normalizer_size)
        self._known = {}  # handle -> (encoded name, element count), dropped on write
        self._names1 = {}  # handle -> one-element ctypes array with its encoded name (fused product of one matrix)
        self.fused_rows = True  # serve single-row linear() calls with the fused decode-and-multiply kernel
        self.group_rows = True  # ... and runs of them that share their activation with one launch
        self._runs = {}         # first handle of a learned run -> (handles, names, rows, biases)
        self._member_of = {}    # the other handles of learned runs -> their first handle
        self._no_run = set()    # first handles whose run did not repeat itself
        self._parked = {}       # handle -> (activation, its version, result, first handle, bias) computed ahead
        self._cur = None        # the run being observed: (activation, its version, [(handle, rows, bias)])
        self._plans = {}        # tuple of handles -> read_batch plan
        cus = torch.cuda.get_device_properties(self._device).multi_processor_count
        self.ahead_fill = 2 * 4 * cus * 64 * 256  # elements that give every SIMD unit two wavefronts
        # dense weights: which handles to decode in the same launch, and the decoded ones that wait
        self._order = RequestOrder(self._decode_one, self._decode_many, lambda h: self._meta(h)[1],
                                   self.ahead_fill, self._MAX_AHEAD)

    def close(self):
        self._held = []
        if getattr(self, "_h", None) is not None and self._h:
            self._raw.nz_manager_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _dtype_code(t: torch.Tensor) -> int:
        if t.dtype == torch.bfloat16:
            return _lib.DTYPE_BF16
        # cuda/high_level.cu:159-161
        raise RuntimeError("Unsupported data type")

    def write(self, handle: str, tensor: torch.Tensor) -> None:
        if not tensor.is_cuda:  # cuda/high_level.cu:133-135
            tensor = tensor.to(self._device)
        code = self._dtype_code(tensor)
        flat = tensor.detach().contiguous().view(-1)
        copied = flat.data_ptr() % 16 != 0
        if copied:
            flat = flat.clone()
        self._stored_anew(handle)
        stream = torch.cuda.current_stream(flat.device)
        if (self.write_behind and 0 < flat.numel() <= self.ahead_fill // 4 and flat.device == self._device
                and not torch.cuda.is_current_stream_capturing()):
            # A tensor this small is a few dozen workgroups and its encode takes as long as
            # that of one sixteen times its size: keep a copy (the caller may change or free
            # the tensor as soon as this call returns) and store it together with the writes
            # that follow, at the latest before the next call that looks at the store.
            self._held = [w for w in self._held if w[0] != handle]
            self._held.append((handle, flat if copied else flat.clone(), stream))
            self._held_elems = sum(w[1].numel() for w in self._held)
            if len(self._held) >= 16 or self._held_elems >= self.ahead_fill:
                self.flush()
            return
        rc = self._L.nz_manager_write(self._h, handle.encode(), flat.data_ptr(), flat.numel(), code,
                                      stream.cuda_stream)
        # A write into existing buffers returns while the encode kernel is still reading `flat`.
        # Memory that came from another stream's pool must not go back to it before then.
        if rc == 0 and flat.numel():
            flat.record_stream(stream)
        _lib.raise_for(rc)

    def flush(self) -> None:
        """Store the writes that are held back (one launch), on the current stream."""
        if not self._held:
            return
        if torch.cuda.is_current_stream_capturing():
            # the call that asks for this is refused as a whole; the writes stay held
            raise ValueError("writes are held back and cannot be stored while the stream is being captured")
        held, self._held, self._held_elems = self._held, [], 0
        now = torch.cuda.current_stream(self._device)
        for _, t, made_on in held:
            if made_on != now:
                now.wait_stream(made_on)
                t.record_stream(now)
        try:
            self.write_batch([h for h, _, _ in held], [t for _, t, _ in held], _told=True)
        except Exception:
            # nothing is lost: they are stored again (writing one twice is harmless) with the next call
            self._held = held + self._held
            self._held_elems = sum(w[1].numel() for w in self._held)
            raise

    def write_batch(self, handles, tensors, _told: bool = False) -> None:
        """Several writes with one host synchronisation (16 per native call).
        (``_told``: the caches have heard of these writes when they were made.)"""
        flats = []
        for t in tensors:
            if not t.is_cuda:
                t = t.to(self._device)
            self._dtype_code(t)
            f = t.detach().contiguous().view(-1)
            flats.append(f.clone() if f.data_ptr() % 16 else f)
        for at in range(0, len(handles), 16):
            hs, fs = handles[at:at + 16], flats[at:at + 16]
            k = len(hs)
            if not _told:
                for h in hs:
                    self._stored_anew(h)
            names = (ctypes.c_char_p * k)(*[h.encode() for h in hs])
            ptrs = (ctypes.c_void_p * k)(*[f.data_ptr() for f in fs])
            ns = (ctypes.c_uint64 * k)(*[f.numel() for f in fs])
            stream = torch.cuda.current_stream(self._device)
            rc = self._L.nz_manager_write_batch(self._h, names, ptrs, ns, k, _lib.DTYPE_BF16, stream.cuda_stream)
            for f in fs:  # see write(): the kernel may still be reading them
                if rc == 0 and f.numel():
                    f.record_stream(stream)
            _lib.raise_for(rc)

    def _stored_anew(self, handle: str) -> None:
        """``handle`` is about to hold other values: nothing derived from the old ones survives"""
        self._known.pop(handle, None)
        self._parked.clear()  # products computed ahead from the weights as they were
        self._order.written(handle)
        if any(handle in key for key in self._plans):  # a plan holds the element counts of its tensors
            self._plans = {key: plan for key, plan in self._plans.items() if handle not in key}

    def _meta(self, handle: str):
        """(encoded name, element count) of a stored handle"""
        known = self._known.get(handle)
        if known is None:
            n = ctypes.c_uint64()
            dt = ctypes.c_int()
            name = handle.encode()
            _lib.raise_for(self._L.nz_manager_meta(self._h, name, ctypes.byref(n), ctypes.byref(dt)))
            known = self._known[handle] = (name, int(n.value))
        return known

    def read(self, handle: str) -> torch.Tensor:
        name, numel = self._meta(handle)
        out = torch.empty(numel, dtype=torch.bfloat16, device=self._device)
        rc = self._L.nz_manager_read(self._h, name, out.data_ptr(), numel, _stream_ptr(self._device))
        _lib.raise_for(rc)
        return out

    def numel(self, handle: str) -> int:
        n = ctypes.c_uint64()
        _lib.raise_for(self._L.nz_manager_meta(self._h, handle.encode(), ctypes.byref(n), None))
        return int(n.value)

    def geometry(self, handle: str):
        """(elements per frequency table, symbols per rANS lane and segment) the entry was written with"""
        c, l = ctypes.c_uint32(), ctypes.c_uint32()
        _lib.raise_for(self._L.nz_manager_geometry(self._h, handle.encode(), ctypes.byref(c), ctypes.byref(l)))
        return int(c.value), int(l.value)

    @property
    def size_budget(self) -> float:
        """stored exponent bytes over their order-0 entropy that the manager's geometry choices keep to"""
        return float(self._L.nz_manager_size_budget(self._h))

    def estimated_size_ratio(self, numel: int, chunk_size: int, lane_symbols: int) -> float:
        """the library's estimate of that ratio for a tensor of ``numel`` elements (0 for an invalid geometry)"""
        return float(self._L.nz_estimated_size_ratio(numel, chunk_size, lane_symbols))

    def in_budget(self, numel: int, chunk_size: int, lane_symbols: int) -> bool:
        """whether the manager's own choices would accept this geometry for a tensor of ``numel`` elements"""
        return bool(self._L.nz_manager_in_budget(self._h, numel, chunk_size, lane_symbols))

    def geometry_hint(self, handle: str, chunk_size: int, lane_symbols: int) -> None:
        """The next writes under ``handle`` use this geometry; (0, 0) takes the hint back."""
        _lib.raise_for(self._L.nz_manager_geometry_hint(self._h, handle.encode(), chunk_size, lane_symbols))

    def read_into(self, handle: str, out: torch.Tensor) -> torch.Tensor:
        """Decompress into caller-provided bf16 storage (no allocation), on the current stream."""
        if out.dtype != torch.bfloat16 or not out.is_contiguous():
            raise ValueError("read_into needs a contiguous bfloat16 tensor")
        rc = self._L.nz_manager_read(self._h, handle.encode(), out.data_ptr(), out.numel(),
                                     _stream_ptr(out.device))
        _lib.raise_for(rc)
        return out

    def batch_plan(self, handles):
        """Argument block for :meth:`read_batch` over a fixed list of handles
        (built once, reused for every call)."""
        k = len(handles)
        names = (ctypes.c_char_p * k)(*[h.encode() for h in handles])
        caps = (ctypes.c_uint64 * k)(*[self.numel(h) for h in handles])
        return names, caps, k

    def read_batch(self, plan, outs) -> None:
        """Decompress the planned handles into the bf16 tensors ``outs`` with one
        kernel launch on the current stream (no allocation, no host sync)."""
        names, caps, k = plan
        if len(outs) != k:
            raise ValueError("one output tensor per planned handle")
        for i, o in enumerate(outs):
            if o.dtype != torch.bfloat16 or not o.is_contiguous() or o.numel() < caps[i]:
                raise ValueError("read_batch needs contiguous bfloat16 outputs of the stored sizes")
        ptrs = (ctypes.c_void_p * k)(*[o.data_ptr() for o in outs])
        rc = self._L.nz_manager_read_batch(self._h, names, ptrs, caps, k, _stream_ptr(outs[0].device) if k else None)
        _lib.raise_for(rc)

    def gather_rows(self, handle: str, indices: torch.Tensor, row_len: int) -> torch.Tensor:
        """Rows ``indices`` (any integer shape) of the stored table with rows of
        ``row_len`` elements -> ``[indices.numel(), row_len]``; only the chunks
        that hold those rows are decoded."""
        idx = indices.reshape(-1).to(device=self._device, dtype=torch.int64).contiguous()
        out = torch.empty(idx.numel(), row_len, dtype=torch.bfloat16, device=self._device)
        rc = self._L.nz_manager_gather_rows(self._h, handle.encode(), idx.data_ptr(), idx.numel(), row_len,
                                            out.data_ptr(), _stream_ptr(self._device))
        _lib.raise_for(rc)
        return out

    def gemv_batch(self, names, x: torch.Tensor, biases, outs, rows: int = 1) -> None:
        """``outs[i] = x @ W_i^T (+ biases[i])`` for the stored matrices ``names``
        (a ctypes array of encoded handles) and ``rows`` (1..8) activation rows
        ``x`` (contiguous, ``rows * in_features`` values; ``outs[i]`` holds
        ``rows`` contiguous rows of ``out_features_i``); the weights are decoded
        inside the kernel, once, and never written out."""
        k = len(names)
        if x.dtype != torch.bfloat16 or not x.is_contiguous() or rows < 1 or x.numel() % rows:
            raise ValueError("gemv_batch needs contiguous bfloat16 activation rows")
        ys = (ctypes.c_void_p * k)(*[o.data_ptr() for o in outs])
        bs = None
        if biases is not None and any(b is not None for b in biases):
            bs = (ctypes.c_void_p * k)(*[None if b is None else b.data_ptr() for b in biases])
        rc = self._L.nz_manager_gemv_rows_batch(self._h, names, k, x.data_ptr(), rows, x.numel() // rows, bs, ys,
                                                _stream_ptr(x.device))
        _lib.raise_for(rc)

    def export(self, handle: str):
        """The stored streams of an entry as CPU uint8 tensors (container, packed, normalizer bytes)."""
        name = handle.encode()
        if self._L.nz_manager_meta(self._h, name, None, None):
            _lib.raise_for(_lib.ERR_NOT_FOUND)
        comp = torch.empty(self.exp_bytes(handle), dtype=torch.uint8)
        packed = torch.empty(self.packed_bytes(handle), dtype=torch.uint8)
        norm = torch.empty(int(self._L.nz_manager_norm_bytes(self._h, name)), dtype=torch.uint8)
        rc = self._L.nz_manager_export(self._h, name, comp.data_ptr(), comp.numel(), packed.data_ptr(),
                                       packed.numel(), norm.data_ptr() if norm.numel() else None, norm.numel(),
                                       _stream_ptr(self._device))
        _lib.raise_for(rc)
        return comp, packed, norm

    def import_(self, handle: str, comp: torch.Tensor, packed: torch.Tensor, norm: torch.Tensor = None) -> None:
        """Store streams produced by :meth:`export` (checked against this manager's settings)."""
        comp = comp.detach().to("cpu", torch.uint8).contiguous()
        packed = packed.detach().to("cpu", torch.uint8).contiguous()
        norm = torch.empty(0, dtype=torch.uint8) if norm is None else norm.detach().to("cpu", torch.uint8).contiguous()
        self._stored_anew(handle)
        rc = self._L.nz_manager_import(self._h, handle.encode(), comp.data_ptr(), comp.numel(),
                                       packed.data_ptr() if packed.numel() else None, packed.numel(),
                                       norm.data_ptr() if norm.numel() else None, norm.numel(),
                                       _stream_ptr(self._device))
        _lib.raise_for(rc)

    def size(self, handle: str, reference_accounting: bool = False) -> int:
        fn = self._L.nz_manager_size_reference if reference_accounting else self._L.nz_manager_size
        return int(fn(self._h, handle.encode()))

    def exp_bytes(self, handle: str) -> int:
        return int(self._L.nz_manager_exp_bytes(self._h, handle.encode()))

    def packed_bytes(self, handle: str) -> int:
        return int(self._L.nz_manager_packed_bytes(self._h, handle.encode()))

    def trim(self) -> None:
        self._order.clear()
        _lib.raise_for(self._L.nz_manager_trim(self._h))

    def rewrite_stats(self):
        """(write batches encoded in place, entries that outgrew their buffer and were re-placed)"""
        a, b = ctypes.c_uint64(), ctypes.c_uint64()
        _lib.raise_for(self._L.nz_manager_rewrite_stats(self._h, ctypes.byref(a), ctypes.byref(b), None))
        return int(a.value), int(b.value)

    def placed_again(self) -> int:
        """Entries written in place whose records a second kernel had to place
        (a workgroup of the encode kernel gave up waiting for its predecessors)."""
        c = ctypes.c_uint64()
        _lib.raise_for(self._L.nz_manager_rewrite_stats(self._h, None, None, ctypes.byref(c)))
        return int(c.value)

    def check(self) -> None:
        outside, self._outside = getattr(self, "_outside", None), None
        _lib.raise_for(self._L.nz_manager_check(self._h, _stream_ptr(self._device)))
        if outside is not None and bool(outside):
            raise RuntimeError("a row gather was given an index outside the table")

    def note_outside(self, flag: torch.Tensor) -> None:
        """Keeps a device-side flag (no synchronisation) for the next check()."""
        prev = getattr(self, "_outside", None)
        self._outside = flag if prev is None else prev | flag

    # -- one to eight activation rows: decode fused into the product -------------
    #
    # Linears that are called back to back with the very same activation (q/k/v,
    # gate/up) are served by ONE launch, without the caller saying so: the first
    # time such a run of calls is seen it is executed call by call and remembered
    # under its first handle; from then on a call of that handle computes the
    # whole run and parks the other results, which the calls that follow pick up
    # if - and only if - they come with the same tensor object, unmodified, and
    # the same bias.  A run that does not repeat itself is forgotten for good.

    _MAX_RUN = 8
    _MAX_ROWS = 8  # activation rows one launch multiplies with (NZ_GEMV_MAX_ROWS)

    def _fused_ok(self, inputs: torch.Tensor, shape, bias) -> bool:
        if (not self.fused_rows or inputs.dim() == 0 or len(shape) != 2 or inputs.shape[-1] != shape[1]
                or shape[1] % 512 or not 1 <= inputs.numel() // shape[1] <= self._MAX_ROWS
                or inputs.dtype != torch.bfloat16 or not inputs.is_cuda
                or (torch.is_grad_enabled() and inputs.requires_grad)):
            return False
        if inputs.numel() != shape[1] and self._normalizer:
            return False  # several rows per launch are not built for normalized tensors
        if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_cuda or bias.numel() != shape[0]
                                 or not bias.is_contiguous() or (torch.is_grad_enabled() and bias.requires_grad)):
            return False
        return True

    def _forget_run(self, leader: str) -> None:
        self._runs.pop(leader, None)
        self._no_run.add(leader)
        for h in [h for h, first in self._member_of.items() if first == leader]:
            del self._member_of[h]
        for h in [h for h, hit in self._parked.items() if hit[3] == leader]:
            del self._parked[h]

    def _observe(self, handle: str, inputs: torch.Tensor, rows: int, bias) -> None:
        """one more call that was served on its own: does it continue the current run?"""
        cur = self._cur
        if (cur is not None and cur[0] is inputs and cur[1] == inputs._version and len(cur[2]) < self._MAX_RUN
                and all(h != handle for h, _, _ in cur[2])):
            cur[2].append((handle, rows, bias))
            return
        self._close_run()
        self._cur = (inputs, inputs._version, [(handle, rows, bias)])

    def _close_run(self) -> None:
        cur, self._cur = self._cur, None
        if cur is None or len(cur[2]) < 2:
            return
        leader = cur[2][0][0]
        if leader in self._no_run or any(h in self._runs or h in self._member_of for h, _, _ in cur[2]):
            return
        handles = [h for h, _, _ in cur[2]]
        self._runs[leader] = (handles, (ctypes.c_char_p * len(handles))(*[h.encode() for h in handles]),
                              [r for _, r, _ in cur[2]], [b for _, _, b in cur[2]])
        for h in handles[1:]:
            self._member_of[h] = leader

    def _fused_row(self, handle: str, inputs: torch.Tensor, shape, bias):
        """``x @ W^T (+ b)`` for one to eight activation rows without writing the
        dense weight: the product is formed while the weight is decoded
        (nz_manager_gemv_rows_batch).  -> None when the call does not qualify (more
        rows, a row length that is not a multiple of 512, another dtype, a bias the
        kernel cannot take)."""
        if not self._fused_ok(inputs, shape, bias):
            return None
        parked = self._parked.pop(handle, None)
        if parked is not None:
            x0, version, out, leader, b0 = parked
            if x0 is inputs and version == inputs._version and b0 is bias:
                return out.view(*inputs.shape[:-1], shape[0])
            self._forget_run(leader)  # the run did not repeat itself
        x = inputs if inputs.is_contiguous() else inputs.contiguous()
        if x.data_ptr() % 16:
            x = x.clone()
        m_rows = x.numel() // shape[1]
        run = self._runs.get(handle) if self.group_rows else None
        if run is not None:
            handles, names, rows, biases = run
            if biases[0] is bias:
                self._close_run()
                flat = torch.empty(m_rows * sum(rows), dtype=torch.bfloat16, device=x.device)
                outs, at = [], 0
                for r in rows:
                    outs.append(flat[at:at + m_rows * r])
                    at += m_rows * r
                try:
                    self.gemv_batch(names, x, biases, outs, m_rows)
                except (ValueError, RuntimeError):
                    self._forget_run(handle)  # e.g. scratch that cannot grow while a graph is captured
                else:
                    for h, o, b in zip(handles[1:], outs[1:], biases[1:]):
                        self._parked[h] = (inputs, inputs._version, o, handle, b)
                    return outs[0].view(*inputs.shape[:-1], shape[0])
            else:
                self._forget_run(handle)
        names = self._names1.get(handle)
        if names is None:
            names = self._names1[handle] = (ctypes.c_char_p * 1)(handle.encode())
        out = torch.empty(m_rows * shape[0], dtype=torch.bfloat16, device=x.device)
        self.gemv_batch(names, x, [bias], [out], m_rows)
        if self.group_rows and handle not in self._member_of:
            self._observe(handle, inputs, shape[0], bias)
        return out.view(*inputs.shape[:-1], shape[0])

    # -- dense weights: the handles that are asked for next share the launch -----
    #
    # A model asks for its weights in the same order pass after pass, and matrices
    # of a few million elements cannot fill the device on their own: a request
    # that finds nothing waiting decodes, in the same launch, the handles that the
    # learned order (neuzip_amd/_ahead.py) expects next, and those wait for their
    # requests.  A weight that waits is dropped when its handle is written, so what
    # is handed out always equals a decode at the time of the request.  Requests
    # made while a stream is being captured take no part in any of this.

    _MAX_AHEAD = 16  # tensors one decode launch takes (NZ_BATCH_MAX)

    @property
    def decode_ahead(self) -> bool:
        return self._order.enabled

    @decode_ahead.setter
    def decode_ahead(self, on: bool) -> None:
        self._order.enabled = bool(on)
        if not on:
            self._order.clear()

    def _decode_one(self, handle: str):
        return self.read(handle), torch.cuda.current_stream(self._device)

    def _decode_many(self, handles):
        """one launch for ``handles`` (a handle may appear twice) -> [(flat weight, stream)], or None"""
        key = tuple(handles)
        plan = self._plans.get(key)
        if plan is None:
            plan = self._plans[key] = self.batch_plan(handles)
        sizes = [int(c) for c in plan[1]]
        flat = torch.empty(sum((n + 7) & ~7 for n in sizes), dtype=torch.bfloat16, device=self._device)
        outs, at = [], 0
        for n in sizes:
            outs.append(flat[at:at + n])
            at += (n + 7) & ~7
        try:
            self.read_batch(plan, outs)
        except (ValueError, RuntimeError):  # e.g. scratch that cannot grow
            self._plans.pop(key, None)
            return None
        stream = torch.cuda.current_stream(self._device)
        return [(o, stream) for o in outs]

    def _dense_weight(self, handle: str) -> torch.Tensor:
        """the decoded weight of ``handle`` (flat), possibly a view of a buffer it shares with its neighbours"""
        if torch.cuda.is_current_stream_capturing():
            # a weight that waits across the end of a capture would be memory of the graph's
            # pool that no kernel has filled yet, and one decoded before the capture would be
            # baked into the graph by address: a captured request decodes its own tensor
            self._order.clear()
            self._order.forget_position()
            return self.read(handle)
        (w, decoded_on), ahead = self._order.request(handle)
        if ahead:
            now = torch.cuda.current_stream(self._device)
            if now != decoded_on:
                now.wait_stream(decoded_on)
                w.record_stream(now)
        return w

    def read_shared(self, handle: str) -> torch.Tensor:
        """The decoded weight for a caller that only reads it and drops it at once."""
        return self._dense_weight(handle)

    def ahead_stats(self):
        """(weights decoded ahead that were asked for, weights decoded ahead and dropped unused)"""
        return self._order.hits, self._order.waste

    def _weight_for_gemm(self, handle: str, inputs: torch.Tensor, shape, bias) -> torch.Tensor:
        """The dense weight of ``handle`` for a call with more rows than the fused
        product takes.  The runs of Linears that share their activation are learned
        here as well (for the calls with few rows that may follow)."""
        if (self.group_rows and self.fused_rows and inputs.is_cuda and len(shape) == 2
                and not (torch.is_grad_enabled() and inputs.requires_grad)):
            if handle in self._runs:
                self._close_run()
            elif handle not in self._member_of:
                self._observe(handle, inputs, shape[0], bias)
        return self._dense_weight(handle).view(shape)

    def linear(self, handle: str, inputs: torch.Tensor, shape, bias: torch.Tensor) -> torch.Tensor:
        # cuda/high_level.cu:252-257: addmm(bias, input, W^T).  The reference only
        # accepts a 2-D input here; inputs with leading batch dimensions take
        # the equivalent F.linear route.  One to eight activation rows (single-token
        # inference, a small batch) are served by the fused decode-and-multiply kernel.
        fused = self._fused_row(handle, inputs, shape, bias)
        if fused is not None:
            return fused
        weight = self._weight_for_gemm(handle, inputs, shape, bias)
        if inputs.dim() == 2:
            return torch.addmm(bias, inputs, weight.t())
        return torch.nn.functional.linear(inputs, weight, bias)

    def linear_without_bias(self, handle: str, inputs: torch.Tensor, shape) -> torch.Tensor:
        # cuda/high_level.cu:259-263
        fused = self._fused_row(handle, inputs, shape, None)
        if fused is not None:
            return fused
        weight = self._weight_for_gemm(handle, inputs, shape, None)
        return torch.matmul(inputs, weight.t())

    def split(self, tensor: torch.Tensor):
        if not tensor.is_cuda:  # cuda/high_level.cu:302-304
            tensor = tensor.to(self._device)
        self._dtype_code(tensor)
        flat = tensor.detach().contiguous().view(-1)
        if flat.data_ptr() % 16:
            flat = flat.clone()
        n = flat.numel()
        exps = torch.empty(n, dtype=torch.uint8, device=flat.device)
        fracs = torch.empty(n, dtype=torch.uint8, device=flat.device)
        norm = None
        if self._normalizer:  # scratch: the reference computes the group bytes and drops them (high_level.cu:282-296)
            norm = torch.empty(self._L.nz_norm_bytes(n, self._normalizer) + 8, dtype=torch.uint8, device=flat.device)
        rc = self._L.nz_split(flat.data_ptr(), n, exps.data_ptr(), fracs.data_ptr(), self._normalizer,
                              norm.data_ptr() if norm is not None else None, _stream_ptr(flat.device))
        _lib.raise_for(rc)
        return [exps, fracs]


class _DenseBackend:
    """Uncompressed pass-through selected by ``Algorithm.dummy``
    (the reference's DummyBackend, neuzip/binding.py:35-52)."""

    def __init__(self):
        self._store = {}

    def write(self, handle: str, tensor: torch.Tensor) -> None:
        self._store[handle] = tensor.cuda()

    def read(self, handle: str) -> torch.Tensor:
        return self._store[handle]

    def size(self, handle: str, reference_accounting: bool = False) -> int:
        t = self._store[handle]
        return t.numel() * t.element_size()

    def linear(self, handle: str, inputs: torch.Tensor, shape, bias=None) -> torch.Tensor:
        with torch.no_grad():
            return torch.nn.functional.linear(inputs, self.read(handle).reshape(shape), bias)

    linear_without_bias = linear


class Manager:
    """Handle-keyed store of compressed tensors (neuzip/binding.py:55-115).

    ``write`` returns the handle (auto-numbered ``"0"``, ``"1"``, ... when none
    is given), ``read`` hands back a fresh dense tensor of the original shape,
    ``linear`` computes ``x @ W^T (+ b)`` against the stored weight and
    ``convert`` swaps the Linear layers of a model in place.
    """

    def __init__(
        self,
        algorithm: Algorithm = Algorithm.ans,
        precision: int = 7,
        normalizer_size=None,
        chunk_size=None,
        lane_symbols: int = 0,
        size_budget: Optional[float] = None,
    ) -> None:
        """``chunk_size`` is the number of exponents that share one frequency
        table.  The reference passes its value (default ``2**16``) to nvcomp as
        the chunk size; here ``None`` selects the library's own table scope of
        ``2**17`` elements decoded by eight wavefronts, which is both smaller and
        faster on this hardware, and ``2**16`` (or any supported value) is
        honoured when given.  ``lane_symbols`` (extension; 0 = the shortest
        segments that stay inside the size budget for the chunk) is the number of
        exponents each of the 64 rANS lanes of a wavefront codes per segment:
        smaller values expose more wavefronts per chunk at the price of about
        4.5 bits of container per lane and segment.  ``"auto"`` picks the
        geometry per tensor from its size and from how many decode workgroups
        the device holds at once, inside the size budget.  ``size_budget``
        (extension; default 1.01) bounds what the manager's own geometry choices
        may store for the exponents, as a multiple of their order-0 entropy
        (estimated from the geometry): at the default, small tensors keep the
        default geometry and are best served by the calls that take several
        tensors per launch (``write_many``, ``DecompressAhead``, ``FusedGemv``);
        a larger budget lets ``"auto"`` give them shorter segments so that each
        of them fills the GPU on its own."""
        normalizer_size = 0 if normalizer_size is None else normalizer_size
        self.meta_dict = {}  # handle -> original shape
        self._stamps = {}    # handle -> number of writes: lets caches of decoded weights notice
        self._on_write = None  # called with the handle before a write is enqueued (decode-ahead hooks in here)
        if algorithm == Algorithm.dummy:
            self._be = _DenseBackend()
            return
        if algorithm != Algorithm.ans:
            # the reference builds an nvcomp manager for these (cuda/high_level.cu:52-65);
            # nvcomp does not exist on this platform
            raise RuntimeError("Unsupported algorithm")
        if precision not in (0, 1, 3, 7) or normalizer_size not in _VALID_NORMALIZERS:
            # the reference resolves a class by name and fails the same way (binding.py:69-70)
            raise AttributeError(
                f"module 'neuzip._cuda' has no attribute 'Manager_f{precision}_n{normalizer_size}'"
            )
        self._be = _HipBackend(precision, normalizer_size, int(chunk_size or 0), lane_symbols, size_budget)
        # what a checkpoint must agree on (the chunk geometry travels inside every container)
        self._settings = {"precision": int(precision), "normalizer_size": int(normalizer_size)}

    # -- store ---------------------------------------------------------------
    def _note_write(self, handle: str) -> None:
        self._stamps[handle] = self._stamps.get(handle, 0) + 1
        if self._on_write is not None:
            self._on_write(handle)

    def write(self, tensor: torch.Tensor, handle: Optional[str] = None) -> str:
        key = str(len(self.meta_dict)) if handle is None else handle
        self.meta_dict[key] = tensor.shape
        self._note_write(key)
        self._be.write(key, tensor)  # note the argument order of the backend
        return key

    def write_many(self, tensors, handles) -> None:
        """``write`` for several (tensor, handle) pairs with one host
        synchronisation per 16 tensors instead of one per tensor (no
        counterpart in the reference)."""
        tensors, handles = list(tensors), list(handles)
        if len(tensors) != len(handles) or len(set(handles)) != len(handles):
            raise ValueError("one distinct handle per tensor")
        for t, h in zip(tensors, handles):
            self.meta_dict[h] = t.shape
            self._note_write(h)
        if hasattr(self._be, "write_batch"):
            self._be.write_batch(handles, tensors)
        else:
            for t, h in zip(tensors, handles):
                self._be.write(h, t)

    def read(self, handle: str) -> torch.Tensor:
        """The stored tensor, decompressed (neuzip/binding.py:88-92).  With
        ``decode_ahead`` the result may be a view into a buffer it shares with the
        weights that are expected to be asked for next: its own part of it, free to
        be changed in place, but ``clone()`` it before serialising it or keeping it
        for long (the view keeps the whole buffer alive)."""
        shape = self.meta_dict[handle]  # KeyError for an unknown handle, as in the reference
        be = self._be
        flat = be.read_shared(handle) if getattr(be, "decode_ahead", False) else be.read(handle)
        return flat.requires_grad_(False).reshape(shape)

    def read_shared(self, handle: str) -> torch.Tensor:
        """Like ``read``, but the result may be a view of a buffer that the next
        call on this manager reuses: for callers that only read the weight and
        drop it at once (the backward pass of a compressed Linear)."""
        if hasattr(self._be, "read_shared"):
            return self._be.read_shared(handle).requires_grad_(False).reshape(self.meta_dict[handle])
        return self.read(handle)

    def size(self, handle: str, reference_accounting: bool = False) -> int:
        """Bytes held for ``handle``: exponent container + stored sign|mantissa
        bytes + normalizer bytes (0 for an unknown handle).  The reference also
        counts a buffer of ``ceil(numel / 1024)`` bytes that it allocates and
        never uses when normalizers are off (cuda/high_level.cu:89-93,208-221);
        ``reference_accounting=True`` adds those bytes, so that the figure
        follows the reference's formula term by term."""
        return self._be.size(handle, reference_accounting)

    def linear(self, handle: str, inputs: torch.Tensor, bias=None) -> torch.Tensor:
        """``inputs @ W^T (+ bias)`` against the stored weight (neuzip/binding.py:97-102).
        One to eight activation rows of a multiple of 512 elements (single-token
        inference, a small batch, a speculative step) are multiplied while the
        weight is decoded, without the dense weight ever being written; its sums are formed in an order of their own, so the
        result agrees with the decompress-then-GEMM path to rounding, not bit for
        bit (``manager.fused_rows = False`` keeps every call on that path).
        Such calls that come back to back with the same activation tensor (q/k/v,
        gate/up) are recognised when they first occur and share one launch from
        then on (``manager.group_rows = False`` turns that off); the numbers are
        those of the single launches."""
        shape = self.meta_dict[handle]
        if bias is None:
            return self._be.linear_without_bias(handle, inputs, shape)
        return self._be.linear(handle, inputs, shape, bias)

    @property
    def fused_rows(self) -> bool:
        return bool(getattr(self._be, "fused_rows", False))

    @fused_rows.setter
    def fused_rows(self, on: bool) -> None:
        if hasattr(self._be, "fused_rows"):
            self._be.fused_rows = bool(on)

    @property
    def group_rows(self) -> bool:
        """Whether single-row calls that arrive back to back with the very same
        activation (q/k/v, gate/up) are learned and served by one launch."""
        return bool(getattr(self._be, "group_rows", False))

    @group_rows.setter
    def group_rows(self, on: bool) -> None:
        if hasattr(self._be, "group_rows"):
            self._be.group_rows = bool(on)

    @property
    def write_behind(self) -> bool:
        """Whether writes of small tensors (up to 8 M elements, a few dozen
        workgroups each) are held back, as a copy made at the time of the call,
        until 16 of them or 33.5 M elements share one encode launch.  Every other
        call on the manager stores them first, so no call can tell the difference;
        ``flush()`` stores them at once."""
        return bool(getattr(self._be, "write_behind", False))

    @write_behind.setter
    def write_behind(self, on: bool) -> None:
        if hasattr(self._be, "write_behind"):
            if not on:
                self._be.flush()
            self._be.write_behind = bool(on)

    def flush(self) -> None:
        """Store the writes that are held back (see ``write_behind``)."""
        if hasattr(self._be, "flush"):
            self._be.flush()

    @property
    def decode_ahead(self) -> bool:
        """Whether a request for a dense weight (a ``linear`` call with many rows,
        the backward pass of a compressed Linear) also decodes, in the same launch,
        the weights that were asked for next the last time round, until the launch
        fills the device.  What is handed out always equals a decode at the time
        of the request: a write drops the weight that waits for its handle.  Turns
        itself off on a manager whose requests do not repeat their order."""
        return bool(getattr(self._be, "decode_ahead", False))

    @decode_ahead.setter
    def decode_ahead(self, on: bool) -> None:
        if hasattr(self._be, "decode_ahead"):
            self._be.decode_ahead = bool(on)

    def gather_rows(self, handle: str, indices: torch.Tensor) -> torch.Tensor:
        """Rows ``indices`` of the stored 2-D table ``handle`` as ``[indices.numel(), row_len]``
        (no counterpart in the reference, which decompresses the whole table:
        neuzip/nn/embedding.py:30-39)."""
        shape = self.meta_dict[handle]
        if len(shape) != 2:
            raise ValueError("gather_rows needs a stored 2-D table")
        if isinstance(self._be, _DenseBackend):
            return self._be.read(handle).reshape(shape)[indices.reshape(-1)]
        # Every requested row decodes the chunk(s) it lies in.  Once that is as much
        # work as decoding the table, do what the reference does: the whole table
        # once, then an ordinary index (neuzip/nn/embedding.py:30-39).
        rows, row_len = int(shape[0]), int(shape[1])
        chunk, _ = self._be.geometry(handle)
        per_row = 1 if (row_len <= chunk and chunk % row_len == 0) else (row_len + chunk - 2) // chunk + 1
        n_chunks = -(-rows * row_len // chunk)
        if indices.numel() * per_row >= n_chunks:
            idx = indices.reshape(-1).to(device=self._be._device, dtype=torch.int64)
            outside = (idx < 0) | (idx >= rows)  # as in the row gather: a row of zeros
            out = self.read(handle).index_select(0, idx.clamp(0, rows - 1))
            self._be.note_outside(outside.any())     # reported by check(), as the row gather's are
            return out.masked_fill_(outside.unsqueeze(1), 0)
        return self._be.gather_rows(handle, indices, row_len)

    # -- checkpointing (no counterpart in the reference, whose compressed tensors
    #    live only inside the process: neuzip/nn/module.py:13) ------------------
    def state_dict(self) -> dict:
        """Everything needed to rebuild the store: settings, shapes and, per
        handle, the entropy-coded exponent container and the packed
        sign|mantissa stream as CPU uint8 tensors.  Plain containers and tensors
        only, so ``torch.save`` / ``torch.load(weights_only=True)`` round-trip it."""
        if isinstance(self._be, _DenseBackend):
            raise RuntimeError("the dummy backend holds dense tensors: save the model's own state_dict")
        entries = {}
        for handle, shape in self.meta_dict.items():
            comp, packed, norm = self._be.export(handle)
            entries[handle] = {"shape": [int(d) for d in shape], "container": comp, "packed": packed,
                               "normalizers": norm}
        return {"neuzip_amd_format": _lib.load().nz_abi_version(), **self._settings, "entries": entries}

    def load_state_dict(self, state: dict) -> None:
        """Replace (or add) the entries named in ``state``; handles keep their
        names, so the ``Parameter`` objects of a converted model see the loaded
        weights.  Settings must match the manager's."""
        if state.get("neuzip_amd_format") != _lib.load().nz_abi_version():
            raise RuntimeError("checkpoint was written with another container format version")
        for key, mine in self._settings.items():
            if state.get(key) != mine:
                raise RuntimeError(f"checkpoint has {key}={state.get(key)}, this manager {key}={mine}")
        for handle, ent in state["entries"].items():
            shape = torch.Size(ent["shape"])
            self._note_write(handle)
            self._be.import_(handle, ent["container"], ent["packed"], ent.get("normalizers"))
            if self._be.numel(handle) != shape.numel():
                raise RuntimeError(f"entry {handle!r}: shape {tuple(shape)} does not match the stored element count")
            self.meta_dict[handle] = shape

    def save(self, path) -> None:
        torch.save(self.state_dict(), path)

    def load(self, path) -> None:
        self.load_state_dict(torch.load(path, map_location="cpu", weights_only=True))

    # -- helpers -------------------------------------------------------------
    def convert(self, module: torch.nn.Module) -> torch.nn.Module:
        module = _convert(self, module)
        self.trim()  # the encode workspace of the largest layer is not needed to serve the model
        return module

    def trim(self) -> None:
        """Free the scratch the backend keeps between calls (re-allocated on demand)."""
        if hasattr(self._be, "trim"):
            self._be.trim()

    def split(self, tensor: torch.Tensor):
        exp, frac = self._be.split(tensor)
        return exp.reshape(tensor.shape), frac.reshape(tensor.shape)

    def __del__(self):
        be = self.__dict__.get("_be")
        if be is not None and hasattr(be, "close"):
            be.close()
