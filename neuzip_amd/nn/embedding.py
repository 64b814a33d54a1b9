"""``Embedding``: drop-in for ``torch.nn.Embedding`` with a compressed table.

Counterpart of neuzip/nn/embedding.py:13-39.  The reference decompresses the
whole table on every forward; here only the chunks that hold the looked-up
rows are decoded (``Manager.gather_rows``), which is what a one-token decode
step needs.  Like the reference's, the table is frozen: the lookup carries no
gradient to it.
"""
from __future__ import annotations

import torch

from neuzip_amd.nn.module import Parameter


class Embedding(torch.nn.Module):
    def __init__(self, manager, embedding: torch.nn.Embedding) -> None:
        super().__init__()
        self.manager = manager
        self.num_embeddings = embedding.num_embeddings
        self.embedding_dim = embedding.embedding_dim
        self.padding_idx = embedding.padding_idx
        self.max_norm = embedding.max_norm
        self.norm_type = embedding.norm_type
        self.scale_grad_by_freq = embedding.scale_grad_by_freq
        self.sparse = embedding.sparse
        self._p = Parameter(self.manager, embedding.weight.data)
        # A lookup decodes whole chunks.  With a manager that chooses the geometry
        # per tensor and whose size budget allows them (they store 1.036 x the
        # exponents' entropy, the default budget is 1.01), the table is stored with
        # the shortest segments there are (32 Ki chunks of eight 4 Ki segments): one
        # row of a 128256 x 4096 table then takes 18 us instead of 39, 512 rows 27 us
        # instead of 55, for 0.6 % more stored bytes and a slower read of the whole
        # table (424 against 344 us).
        be = getattr(self.manager, "_be", None)
        if getattr(be, "auto_geometry", False):
            h = self._p._handle
            if be.geometry(h) != (32768, 64) and be.in_budget(self._p._shape.numel(), 32768, 64):
                dense = self.manager.read(h)
                be.geometry_hint(h, 32768, 64)
                self.manager.write(dense, h)

    @property
    def weight(self) -> Parameter:
        return self._p

    def extra_repr(self) -> str:
        # the leading "!" marks a converted layer in the printed module tree
        return (f"! num_embeddings={self.num_embeddings}, embedding_dim={self.embedding_dim}, "
                f"padding_idx={self.padding_idx}, max_norm={self.max_norm}, norm_type={self.norm_type}, "
                f"scale_grad_by_freq={self.scale_grad_by_freq}, sparse={self.sparse}")

    def forward(self, x):
        gather = getattr(self.manager, "gather_rows", None)
        if gather is None or not x.is_cuda:
            table = self._p()
            return torch.nn.functional.embedding(x, table, self.padding_idx, self.max_norm, self.norm_type,
                                                 self.scale_grad_by_freq, self.sparse)
        with torch.no_grad():
            rows = gather(self._p._handle, x)  # [x.numel(), embedding_dim]
            if self.max_norm is None:
                return rows.view(*x.shape, self.embedding_dim)
            # row renormalisation is torch's own: look the gathered rows up by position
            pos = torch.arange(x.numel(), device=rows.device).view(x.shape)
            return torch.nn.functional.embedding(pos, rows, None, self.max_norm, self.norm_type)
