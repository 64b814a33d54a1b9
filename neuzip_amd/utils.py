"""Walk a module tree and swap dense Linear layers for compressed ones.

Counterpart of ``_convert`` in neuzip/utils.py:57-68: children whose attribute
name contains ``lm_head`` are left alone, ``nn.Linear`` (and HuggingFace
``Conv1D`` when transformers is importable) are replaced, everything else is
descended into.  Embeddings are not converted by ``_convert``;
``_unroll_convert`` (neuzip/utils.py:41-54) replaces every Linear AND every
Embedding of the tree, ``lm_head`` included.
"""
from __future__ import annotations

import logging

import torch

logger = logging.getLogger(__name__)


def _convertible_types():
    kinds = [torch.nn.Linear]
    try:  # transformers is optional on this platform
        from transformers.pytorch_utils import Conv1D

        kinds.append(Conv1D)
    except Exception:  # pragma: no cover
        pass
    return tuple(kinds)


def _delete_module(module: torch.nn.Module) -> None:
    """Release the dense parameters of a module that has been replaced."""
    for pname in [n for n, _ in module.named_parameters()]:
        setattr(module, pname, None)


def _set_module_by_name(parent: torch.nn.Module, name: str, child: torch.nn.Module) -> None:
    """``parent.a.3.b = child`` for the dotted ``name`` "a.3.b" (neuzip/utils.py:19-31)."""
    *path, leaf = name.split(".")
    holder = parent
    for part in path:
        holder = holder[int(part)] if part.isnumeric() else getattr(holder, part)
    setattr(holder, leaf, child)


def _unroll_convert(manager, module: torch.nn.Module) -> torch.nn.Module:
    """In place: every ``nn.Linear`` becomes a compressed Linear and every
    ``nn.Embedding`` a compressed Embedding (neuzip/utils.py:41-54)."""
    from neuzip_amd.nn import Embedding, Linear

    for name, m in list(module.named_modules()):
        if not name:
            continue
        if isinstance(m, torch.nn.Linear):
            logger.debug("Quantizing %s: %s", name, m)
            _set_module_by_name(module, name, Linear(manager, m))
            _delete_module(m)
        elif isinstance(m, torch.nn.Embedding):
            logger.debug("Quantizing %s: %s", name, m)
            _set_module_by_name(module, name, Embedding(manager, m))
            _delete_module(m)
    return module


def _convert(manager, module: torch.nn.Module, prefix: str = "") -> torch.nn.Module:
    from neuzip_amd.nn import Linear

    kinds = _convertible_types()
    pending = [(module, prefix)]
    while pending:
        parent, path = pending.pop()
        for name, child in list(parent.named_children()):
            dotted = f"{path}.{name}" if path else name
            if "lm_head" in name:
                continue
            if isinstance(child, kinds):
                logger.debug("Converting %s: %s", dotted, child)
                setattr(parent, name, Linear(manager, child))
                _delete_module(child)
            else:
                pending.append((child, dotted))
    return module
