"""Reader and writer of the single-file safetensors format: an 8-byte
little-endian header length, a JSON header ``name -> {dtype, shape,
data_offsets}``, then the raw bytes. The checks follow the reference's reader
(src/alofa/model/safetensors.mojo:147-303)."""
from __future__ import annotations

import json
import struct
from pathlib import Path

import numpy as np
import torch

from ..errors import AlofaError

# stored dtype -> (numpy dtype that carries the bits, torch dtype of the view)
_STORED = {
    "F32": (np.dtype("<f4"), torch.float32),
    "BF16": (np.dtype("<u2"), torch.bfloat16),
    "I32": (np.dtype("<i4"), torch.int32),
}
_NAMES = {torch.float32: "F32", torch.bfloat16: "BF16", torch.int32: "I32"}


class SafeTensorFile:
    """name -> tensor views into a copy-on-write mapping of the file."""

    def __init__(self, path):
        self.path = Path(path)
        try:
            size = self.path.stat().st_size
            with open(self.path, "rb") as f:
                head = f.read(8)
                if len(head) < 8:
                    raise AlofaError("parse", "file is too short for a safetensors header", f"path={self.path}")
                (n,) = struct.unpack("<Q", head)
                if n == 0:
                    raise AlofaError("parse", "safetensors header is empty", f"path={self.path}")
                if 8 + n > size:
                    raise AlofaError("parse", "safetensors header is longer than the file", f"path={self.path} header={n} size={size}")
                text = f.read(n)
        except OSError as e:
            raise AlofaError("io", "cannot read the weight file", f"path={self.path} reason={e}") from None
        try:
            header = json.loads(text)
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise AlofaError("parse", "safetensors header is not valid JSON", f"path={self.path} reason={e}") from None
        if not isinstance(header, dict):
            raise AlofaError("parse", "safetensors header must be an object", f"path={self.path}")
        header.pop("__metadata__", None)
        self._base = 8 + n
        payload = size - self._base
        self.entries = {}
        for name, e in header.items():
            try:
                dtype, shape, (lo, hi) = e["dtype"], tuple(int(s) for s in e["shape"]), e["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise AlofaError("parse", "malformed tensor entry in the safetensors header", f"name={name}") from None
            if dtype not in _STORED:
                raise AlofaError("unsupported", "tensor dtype is not supported", f"name={name} dtype={dtype}")
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if lo < 0 or hi < lo or (hi - lo) != count * _STORED[dtype][0].itemsize:
                raise AlofaError("parse", "tensor shape does not match its byte range", f"name={name} shape={shape} bytes={hi - lo}")
            if hi > payload:
                raise AlofaError("out_of_range", "tensor lies past the end of the file", f"name={name} end={hi} payload={payload}")
            self.entries[name] = (dtype, shape, lo, hi)
        self._map = np.memmap(self.path, dtype=np.uint8, mode="c", offset=self._base) if payload > 0 else np.zeros(0, np.uint8)

    def names(self):
        return list(self.entries)

    def shape(self, name):
        return self.entries[name][1]

    def stored_dtype(self, name) -> torch.dtype:
        return _STORED[self.entries[name][0]][1]

    def tensor(self, name) -> torch.Tensor:
        """The tensor in its stored dtype; no conversion."""
        if name not in self.entries:
            raise AlofaError("invalid_argument", "parameter is missing", f"name={name}")
        dtype, shape, lo, hi = self.entries[name]
        np_dtype, t_dtype = _STORED[dtype]
        raw = np.asarray(self._map[lo:hi]).view(np_dtype)
        t = torch.from_numpy(raw)
        if t_dtype is torch.bfloat16:
            t = t.view(torch.int16).view(torch.bfloat16)
        return t.reshape(shape)


def write_safetensors(path, tensors: dict) -> None:
    """Write ``name -> tensor`` (float32, bfloat16 or int32, CPU) in the given order."""
    header, offset, blobs = {}, 0, []
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise AlofaError("unsupported", "tensor dtype cannot be written", f"name={name} dtype={t.dtype}")
        t = t.detach().contiguous().cpu()
        raw = (t.view(torch.int16) if t.dtype is torch.bfloat16 else t).numpy().tobytes()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for raw in blobs:
            f.write(raw)
