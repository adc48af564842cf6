"""Face of the C++ host runtime (csrc/host/): loads the library and turns its
negative return codes into named errors."""
from __future__ import annotations

import ctypes

from ..errors import AlofaError
from .build import load_host

_NAMES = {1: "invalid_argument", 2: "out_of_range", 5: "capacity", 11: "double_free"}


def lib() -> ctypes.CDLL:
    return load_host()


def check(rc: int) -> int:
    """A return value >= 0 is handed on; a negative one raises the error it names."""
    if rc >= 0:
        return rc
    text = lib().alofa_host_last_error().decode()
    message, _, detail = text.partition(" [")
    raise AlofaError(_NAMES.get(-rc, "invalid_argument"), message, detail.rstrip("]"))


def int_array(n: int):
    return (ctypes.c_int * max(1, n))()


def long_array(values_or_n):
    if isinstance(values_or_n, int):
        return (ctypes.c_int64 * max(1, values_or_n))()
    return (ctypes.c_int64 * max(1, len(values_or_n)))(*values_or_n)
