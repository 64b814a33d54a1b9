"""Autograd node of a Linear layer whose weight is stored compressed.

Behaviour follows the reference's ``CompressedLinear`` (neuzip/ops/linear.py:11-46):

* forward: honour an active autocast region by casting the activation by hand,
  then ``y = x @ W^T (+ b)`` with ``W`` decompressed just in time and dropped;
* backward: decompress ``W`` a second time for ``dL/dx``, accumulate ``dL/dW``
  on the parameter's ``_gradient`` slot (not in ``.grad``), and hand autograd a
  zero-size tensor for the placeholder so that post-accumulate-grad hooks of
  the compressed parameter still fire.
"""
from __future__ import annotations

import torch


def _as_rows(t: torch.Tensor) -> torch.Tensor:
    """Collapse all leading dimensions: [..., k] -> [m, k]."""
    return t.reshape(-1, t.shape[-1])


class CompressedLinear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inputs, _p, bias):
        ctx._inputs_dtype = inputs.dtype
        x = inputs
        if torch.is_autocast_enabled():
            x = x.to(torch.get_autocast_gpu_dtype())
        ctx.save_for_backward(x, bias)
        ctx.carry = (_p,)
        return _p.linear(x, bias)

    @staticmethod
    def backward(ctx, grad_output):
        x, bias = ctx.saved_tensors
        (_p,) = ctx.carry

        x2d = _as_rows(x)
        go2d = _as_rows(grad_output)
        dense_w = _p.shared()

        grad_x = torch.mm(go2d, dense_w).reshape(x.shape).to(ctx._inputs_dtype)
        del dense_w
        grad_w = torch.mm(go2d.t(), x2d)

        if _p._gradient is None:
            _p._gradient = grad_w
        else:
            _p._gradient.add_(grad_w)

        grad_b = go2d.sum(0) if bias is not None else None
        return grad_x, torch.empty_like(_p.data), grad_b
