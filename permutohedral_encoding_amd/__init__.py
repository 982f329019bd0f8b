"""MI355X-native permutohedral-lattice hash encoding behind the reference's PyTorch surface
(reference: src/__init__.py:6-8)."""
from .modules import PermutoEncoding, Coarse2Fine
from .funcs import PermutoEncodingFunc, PermutoEncodingFuncBack
from .utils import map_range_val, cosine_easing_window

__all__ = ["PermutoEncoding", "Coarse2Fine", "PermutoEncodingFunc", "PermutoEncodingFuncBack", "map_range_val",
           "cosine_easing_window"]
