"""``neuzip.binding`` (neuzip/binding.py:23-115): ``Algorithm`` and ``Manager``
with the reference's constructor defaults, backed by :mod:`neuzip_amd.binding`."""
from neuzip_amd import binding as _b
from neuzip_amd.binding import Algorithm

__all__ = ["Algorithm", "Manager"]


class _ReferenceDefault(int):
    """The reference's default ``chunk_size`` (``2**16``) as the signature shows
    it; as an object of its own it tells a caller who left the argument alone
    from one who asked for 64 Ki chunks."""


_CHUNK_DEFAULT = _ReferenceDefault(2 ** 16)


class Manager(_b.Manager):
    """:class:`neuzip_amd.Manager` with the reference's signature
    (neuzip/binding.py:56-62).  The reference hands ``chunk_size`` to nvcomp as
    its internal unit of work; a caller who leaves it at its default gets what
    serves that purpose here: the library's own table scope, the geometry of
    every tensor chosen from its size inside the size budget of 1.01 (the same
    as ``neuzip_amd.Manager(lane_symbols="auto")``).  An explicit value, 2**16
    included, is honoured as the number of exponents that share a frequency
    table.  Extensions of this build (``lane_symbols``, ``size_budget``) pass
    through as keywords."""

    def __init__(self, algorithm: Algorithm = Algorithm.ans, precision: int = 7, normalizer_size=None,
                 chunk_size=_CHUNK_DEFAULT, **extensions) -> None:
        if chunk_size is _CHUNK_DEFAULT:
            chunk_size = None
            extensions.setdefault("lane_symbols", "auto")
        super().__init__(algorithm=algorithm, precision=precision, normalizer_size=normalizer_size,
                         chunk_size=chunk_size, **extensions)
