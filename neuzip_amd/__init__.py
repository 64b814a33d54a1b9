"""MI355X-native NeuZip.

bf16 weights are held as an rANS-coded exponent stream plus a packed
sign/mantissa stream and are decompressed just in time inside Linear layers.
The public names are those of the reference package (neuzip/__init__.py:8-35).
"""
import torch

from neuzip_amd import nn, ops
from neuzip_amd.binding import Algorithm, Manager
from neuzip_amd.fused import FusedGemv
from neuzip_amd.prefetch import DecompressAhead

__all__ = ["ops", "nn", "Algorithm", "Manager", "DecompressAhead", "FusedGemv", "lomo_hook", "compressed_lomo_hook"]


def _current_lr(scheduler) -> float:
    return scheduler.get_last_lr()[0]


def lomo_hook(scheduler, param):
    """SGD step applied from a post-accumulate-grad hook on a dense parameter
    (neuzip/__init__.py:16-22)."""
    grad = param.grad
    if grad is None:
        return
    with torch.no_grad():
        param.data.add_(grad, alpha=-_current_lr(scheduler))
    param.grad = None


def compressed_lomo_hook(scheduler, param):
    """SGD step on a compressed parameter (neuzip/__init__.py:25-35):
    decompress, ``W -= lr * dW``, re-compress under the same handle, and drop
    the accumulated gradient."""
    grad_w = param._gradient
    if grad_w is None:
        return
    with torch.no_grad():
        dense = param()
        dense.add_(grad_w, alpha=-_current_lr(scheduler))
        param._manager.write(dense, param._handle)
    param._gradient = None
    param.grad = None
