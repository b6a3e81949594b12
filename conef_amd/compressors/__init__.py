"""Count-sketch error compressors (drop-in for the reference's communication/compressors)."""
from .CountSketch import DenseCS  # noqa: F401
from .CountSketchHash3 import DenseCSHash3  # noqa: F401
from . import halfCountSketch  # noqa: F401
