"""``neuzip.binding`` (neuzip/binding.py:23-115): ``Algorithm`` and ``Manager``
with the reference's constructor defaults, backed by :mod:`neuzip_amd.binding`."""
from neuzip_amd import binding as _b
from neuzip_amd.binding import Algorithm

__all__ = ["Algorithm", "Manager"]


class Manager(_b.Manager):
    """:class:`neuzip_amd.Manager` with the reference's signature
    (neuzip/binding.py:56-62): ``chunk_size=2**16`` exponents share one
    frequency table, the unit the reference hands to nvcomp.  Extensions of
    this build (``lane_symbols``) pass through as keywords; ``chunk_size=None``
    selects the library's own, faster table scope of ``2**17``."""

    def __init__(self, algorithm: Algorithm = Algorithm.ans, precision: int = 7, normalizer_size=None,
                 chunk_size=2 ** 16, **extensions) -> None:
        super().__init__(algorithm=algorithm, precision=precision, normalizer_size=normalizer_size,
                         chunk_size=chunk_size, **extensions)
