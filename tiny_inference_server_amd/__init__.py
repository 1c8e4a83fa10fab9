"""A small, whole inference engine for one GPU of the MI355X kind (gfx950), with hand-written HIP kernels."""
__version__ = "0.1.0"

from . import architectures  # noqa: E402,F401  (registers the built-in architectures)
from . import parts          # noqa: E402,F401  (registers the built-in parts)
