"""``Linear``: drop-in for ``torch.nn.Linear`` with a compressed weight.

Counterpart of neuzip/nn/linear.py:14-35: the weight becomes a
:class:`~neuzip_amd.nn.module.Parameter` (exposed as ``.weight`` and stored
under the attribute ``_p``), the bias stays a dense ``nn.Parameter``.
"""
from __future__ import annotations

import torch

from neuzip_amd.nn.module import Parameter
from neuzip_amd.ops import CompressedLinear


class Linear(torch.nn.Module):
    def __init__(self, manager, linear: torch.nn.Linear) -> None:
        super().__init__()
        self.manager = manager
        self.in_features = linear.in_features
        self.out_features = linear.out_features
        if linear.bias is None:
            self.register_parameter("bias", None)
        else:
            self.bias = torch.nn.Parameter(linear.bias.data)
        self._p = Parameter(manager, linear.weight.data)

    @property
    def weight(self) -> Parameter:
        return self._p

    def forward(self, x):
        if not torch.is_grad_enabled():
            # nothing to record for backward: same arithmetic without the autograd node
            if torch.is_autocast_enabled():
                x = x.to(torch.get_autocast_gpu_dtype())
            return self._p.linear(x, self.bias)
        return CompressedLinear.apply(x, self._p, self.bias)

    def extra_repr(self) -> str:
        # the leading "!" marks a converted layer in the printed module tree
        has_bias = self.bias is not None
        return f"! in_features={self.in_features}, out_features={self.out_features}, bias={has_bias}"
