"""MI355X (gfx950) backend for CUT's GGUF quantized-matmul path."""
from . import lib  # noqa: F401
