"""Named errors. The names and numbers follow the reference's list
(src/alofa/core/error.mojo:25-39, :79-108): tests assert on ``err.name``."""
from __future__ import annotations

_CODES = {
    "invalid_argument": 1, "out_of_range": 2, "out_of_memory": 3, "alignment": 4,
    "capacity": 5, "io": 6, "mmap": 7, "unsupported": 8, "shape_mismatch": 9,
    "not_initialized": 10, "double_free": 11, "parse": 12,
}


class AlofaError(Exception):
    """code name + message + detail, printed ``name(code): message [detail]``."""

    def __init__(self, name: str, message: str, detail: str = ""):
        if name not in _CODES:
            raise ValueError(f"unknown error name {name!r}")
        self.name = name
        self.code = _CODES[name]
        self.message = message
        self.detail = detail
        text = f"{name}({self.code}): {message}"
        if detail:
            text += f" [{detail}]"
        super().__init__(text)
