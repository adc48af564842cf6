"""alofa_amd: a small, whole inference engine for one GPU (MI355X, gfx950)."""
from .errors import AlofaError

__all__ = ["AlofaError", "Engine"]
__version__ = "0.1.0"


def __getattr__(name):
    if name == "Engine":
        from .api import Engine
        return Engine
    raise AttributeError(name)
