"""litinfer_amd: a small, whole, one-GPU inference engine for MI355X (gfx950)."""
from . import config, weights, parts, cache  # noqa: F401  (registers architectures and parts)

__version__ = "0.1.0"
