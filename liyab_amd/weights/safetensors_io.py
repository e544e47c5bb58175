"""Reading and writing safetensors files.

The format: 8 bytes little-endian header length, a JSON header
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": ...}`,
then the tensors' bytes. The file is memory-mapped and a tensor is a view of
the map until it is copied to the device, as the reference maps its weights
file and hands out views (`include/liyab/mmap_loader.h:118-139`); malformed
files are refused with what is wrong, as there (`src/core/mmap_loader.cpp`).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Tuple

import numpy as np
import torch

from ..errors import InvalidModel

_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 << 20


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int  # byte offsets within the data section
    end: int


class SafetensorsFile:
    """A memory-mapped safetensors file: `entries` by name, `tensor(name)`."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise InvalidModel(f"not a model folder: '{path}' is missing")
        size = os.path.getsize(path)
        if size < 8:
            raise InvalidModel(f"'{path}' is not a safetensors file: shorter than its header length")
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen < 2 or hlen > _MAX_HEADER or 8 + hlen > size:
            self._f.close()
            raise InvalidModel(f"'{path}' is not a safetensors file: header length {hlen} does not fit the file")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"), object_pairs_hook=_no_duplicates)
        except (UnicodeDecodeError, json.JSONDecodeError, InvalidModel) as e:
            self._f.close()
            raise InvalidModel(f"'{path}': malformed header: {e}") from None
        if not isinstance(header, dict):
            self._f.close()
            raise InvalidModel(f"'{path}': malformed header: not a JSON object")
        self.metadata = header.pop("__metadata__", None) or {}
        self._data_start = 8 + hlen
        data_size = size - self._data_start
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            try:
                dt = info["dtype"]
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                self._f.close()
                raise InvalidModel(f"'{path}': malformed entry for tensor '{name}'") from None
            if dt not in _DTYPES:
                self._f.close()
                raise InvalidModel(f"'{path}': tensor '{name}' has unknown dtype '{dt}'")
            n = 1
            for s in shape:
                if s < 0:
                    self._f.close()
                    raise InvalidModel(f"'{path}': tensor '{name}' has a negative dimension")
                n *= s
            if begin < 0 or end < begin or end > data_size or end - begin != n * _DTYPES[dt][1]:
                self._f.close()
                raise InvalidModel(
                    f"'{path}': tensor '{name}' has offsets [{begin}, {end}) that do not fit its shape "
                    f"{list(shape)} or the file"
                )
            self.entries[name] = TensorEntry(name, _DTYPES[dt][0], shape, begin, end)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor viewing the mapped bytes (read-only: copy before writing)."""
        e = self.entries[name]
        n = e.end - e.begin
        if n == 0:
            return torch.empty(e.shape, dtype=e.dtype)
        buf = np.frombuffer(self._map, dtype=np.uint8, count=n, offset=self._data_start + e.begin)
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the map is not writable
            t = torch.from_numpy(buf)
        return t.view(e.dtype).reshape(e.shape)

    def close(self) -> None:
        # views handed out keep the map alive through numpy's buffer reference
        self._f.close()


def _no_duplicates(pairs):
    out = {}
    for k, v in pairs:
        if k in out:
            raise InvalidModel(f"duplicate tensor name '{k}'")
        out[k] = v
    return out


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] | None = None) -> None:
    """Writes `tensors` (CPU, any of the dtypes above) in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise InvalidModel(f"tensor '{name}' has a dtype safetensors cannot hold: {t.dtype}")
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    hjson = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for raw in blobs:
            f.write(raw)
    os.replace(tmp, path)
