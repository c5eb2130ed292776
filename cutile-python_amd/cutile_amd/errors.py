"""Exception types of the host wrapper.

The reference raises ``TileTypeError`` (src/cuda/tile/_exception.py) for dtype / shape violations
found while typing ``ct.mma_scaled`` and plain ``ValueError`` from its sample wrapper
(samples/BlockScaledMatMul.py:258-264).  The same split is kept here."""


class TileTypeError(TypeError):
    """dtype or shape of an operand violates the rules of ``mma_scaled``."""


class TileValueError(ValueError):
    """An argument value is out of range."""
