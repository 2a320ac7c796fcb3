"""grouped_mm for AMD MI355X (gfx950): drop-in for ``grouped_mm_bf16.grouped_mm``."""
from .api import grouped_mm

__all__ = ["grouped_mm"]
__version__ = "0.1.0"
