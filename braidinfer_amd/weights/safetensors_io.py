"""Reader and writer of the safetensors container, written against the format itself:
8 bytes little-endian header length, a JSON header {name: {dtype, shape, data_offsets}},
then the raw little-endian tensor bytes.  The reference parses the same container with a
crate and mmaps the payload (crates/braidinfer-core/src/safetensors.rs:40-81); sharded
folders go through `model.safetensors.index.json` -> `weight_map` (:102-159).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from typing import Dict, Iterable, List, Tuple

import torch

from ..errors import WeightError

_DTYPES = {
    "BF16": (torch.bfloat16, 2), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I32": (torch.int32, 4), "I64": (torch.int64, 8),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One mmapped .safetensors file; `tensor(name)` is a CPU tensor viewing the map."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise WeightError(f"{path}: cannot open ({e})") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise WeightError(f"{path}: truncated (no header length)")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if 8 + hlen > size:
            raise WeightError(f"{path}: truncated (header of {hlen} bytes in a file of {size})")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError(f"{path}: header is not JSON ({e})") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        self._base = 8 + hlen
        for name, e in header.items():
            dt, shape, (b, en) = e["dtype"], tuple(e["shape"]), e["data_offsets"]
            if dt not in _DTYPES:
                raise WeightError(f"{path}: tensor {name} has unknown dtype {dt}")
            n = 1
            for s in shape:
                n *= s
            if en - b != n * _DTYPES[dt][1] or self._base + en > size:
                raise WeightError(f"{path}: tensor {name} has a bad byte range or the file is truncated")
            self.entries[name] = (dt, shape, b, en)
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        dt, shape, _, _ = self.entries[name]
        return _DTYPES[dt][0], shape

    def tensor(self, name: str) -> torch.Tensor:
        dt, shape, b, e = self.entries[name]
        tdt = _DTYPES[dt][0]
        if e == b:
            return torch.empty(shape, dtype=tdt)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            t = torch.frombuffer(self._mm, dtype=tdt, count=(e - b) // _DTYPES[dt][1], offset=self._base + b)
        return t.reshape(shape)

    def close(self):
        # tensors handed out keep the map alive through the buffer protocol
        self._f.close()


class SafetensorsFolder:
    """All tensors of a model folder: `model.safetensors`, or the shards an index names."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self.files: List[SafetensorsFile] = []
        self.where: Dict[str, SafetensorsFile] = {}
        if os.path.isfile(single):
            paths = [single]
        elif os.path.isfile(index):
            with open(index) as f:
                wm = json.load(f).get("weight_map", {})
            paths = sorted({os.path.join(folder, v) for v in wm.values()})
        else:
            raise WeightError(f"{folder}: neither model.safetensors nor model.safetensors.index.json")
        for p in paths:
            sf = SafetensorsFile(p)
            self.files.append(sf)
            for n in sf.names():
                if n in self.where:
                    raise WeightError(f"{folder}: tensor {n} appears in two files")
                self.where[n] = sf

    def names(self) -> List[str]:
        return list(self.where)

    def info(self, name):
        return self.where[name].info(name)

    def tensor(self, name):
        return self.where[name].tensor(name)


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write CPU tensors in the given order."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blobs = []
    off = 0
    for name, t in tensors:
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise WeightError(f"cannot store dtype {t.dtype} of {name}")
        raw = t.view(torch.uint8).reshape(-1).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
