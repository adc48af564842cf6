"""alofa_amd: a small, whole inference engine for one GPU (MI355X, gfx950)."""
from .errors import AlofaError

__all__ = ["AlofaError"]
__version__ = "0.1.0"
