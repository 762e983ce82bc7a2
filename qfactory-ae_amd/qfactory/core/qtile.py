"""Operand descriptors of a quantized matmul ("QTiles").

Same constructor surface as the reference's ``qfactory/core/qtile.py:1-25``: a tile is a shape, a
storage dtype, a field width in bits and, for quantized operands, the method ("sym" / "asym") and
the granularity of its scales -- ``(1, GS)`` means one scale (and zero-point) per output row and
per GS consecutive elements of K.
"""


class QTile:
    def __init__(self, shape, dtype, nbits, quant_method="none", quant_granularity=None):
        self.shape = tuple(shape)
        self.dtype = dtype
        self.nbits = nbits
        self.quant_method = quant_method
        self.quant_granularity = quant_granularity
        if quant_method == "none":
            return
        if len(self.shape) != len(quant_granularity):
            raise AssertionError("Quantization granularity must match the number of dimensions")
        if quant_granularity[0] != 1:
            raise AssertionError("Scales must be per output row (granularity[0] == 1)")
        for extent, gran in zip(self.shape, quant_granularity):
            if extent % gran != 0:
                raise AssertionError(f"Shape {extent} must be divisible by granularity {gran}")

    @property
    def quantized(self):
        return self.quant_method != "none"

    def __repr__(self):
        q = "" if not self.quantized else f", {self.quant_method}{tuple(self.quant_granularity)}"
        return f"{type(self).__name__}({self.shape}, {self.dtype}, {self.nbits}b{q})"


class SymQTile(QTile):
    """Unsigned storage with the implicit zero-point 2^(b-1); no zero tensor."""

    def __init__(self, shape, dtype, nbits, quant_granularity):
        super().__init__(shape, dtype, nbits, "sym", quant_granularity)


class AsymQTile(QTile):
    """Unsigned storage with a packed per-group zero-point tensor."""

    def __init__(self, shape, dtype, nbits, quant_granularity):
        super().__init__(shape, dtype, nbits, "asym", quant_granularity)
