"""MI355X (gfx950) kernels for AIMET-style quantization simulation behind the aimet_torch API surface.

Importing the package loads ``libmiq.so`` (hand-written HIP kernels behind a C ABI, see ``include/miq.h``); the
import fails if the library has not been built -- there is no CPU or eager-PyTorch compute path.
"""
from . import _lib  # noqa: F401  (loads libmiq.so or raises)

__version__ = "0.1.0"
