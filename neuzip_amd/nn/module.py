"""``Parameter``: the handle a module keeps in place of a dense weight.

Counterpart of neuzip/nn/module.py:11-28.  The tensor data of the parameter is
a zero-element placeholder carrying only dtype and device; the payload lives
in the manager under ``_handle``.  Calling the parameter materialises the dense
weight, ``linear`` runs ``x @ W^T (+ b)`` against it.
"""
from __future__ import annotations

import torch


class Parameter(torch.nn.Parameter):
    def __new__(cls, manager, data, requires_grad=True) -> "Parameter":
        placeholder = torch.zeros(0).to(data)
        self = super().__new__(cls, placeholder, requires_grad)
        self._manager = manager
        self._shape = data.shape
        self._gradient = None
        self._handle = manager.write(data)
        return self

    @torch.no_grad()
    def __call__(self) -> torch.Tensor:
        dense = self._manager.read(self._handle)
        return dense.reshape(self._shape).to(self.device).requires_grad_(False)

    @torch.no_grad()
    def shared(self) -> torch.Tensor:
        """The dense weight for a caller that only reads it and drops it at once
        (may be a view of a buffer the manager reuses)."""
        dense = self._manager.read_shared(self._handle) if hasattr(self._manager, "read_shared") else self()
        return dense.reshape(self._shape)

    def linear(self, inputs, bias=None):
        return self._manager.linear(self._handle, inputs, bias).to(self.device)

    def nbytes_compressed(self) -> int:
        """Bytes the manager holds for this weight."""
        return self._manager.size(self._handle)
