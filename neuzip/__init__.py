"""``import neuzip`` on an MI355X: the reference's package name and surface
(neuzip/__init__.py:8-35) served by :mod:`neuzip_amd`.

``neuzip.Manager().convert(model)``, ``neuzip.nn.*``, ``neuzip.ops.*``,
``neuzip.Algorithm``, ``neuzip.lomo_hook`` and ``neuzip.compressed_lomo_hook``
are the objects of :mod:`neuzip_amd`; the reference's module paths
(``neuzip.utils``, ``neuzip.nn.linear`` ...) resolve to their counterparts.
``neuzip.Manager`` keeps the reference's constructor signature,
``chunk_size=2**16`` included (neuzip/binding.py:56-62); left at that default, every
tensor gets the geometry the library picks for its size.
"""
import sys as _sys

import neuzip_amd as _amd  # raises ImportError when the HIP library is not built (neuzip/binding.py:15-20)
from neuzip_amd import DecompressAhead, FusedGemv, compressed_lomo_hook, lomo_hook, nn, ops, utils

from neuzip.binding import Algorithm, Manager

__all__ = ["ops", "nn", "Algorithm", "Manager"]

# the reference's module paths
for _name in ("utils", "nn", "ops", "nn.linear", "nn.module", "nn.embedding", "ops.linear"):
    _sys.modules[f"{__name__}.{_name}"] = _sys.modules[f"{_amd.__name__}.{_name}"]
del _name
