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
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from ..errors import WeightError

_DTYPES = {
    "BF16": (torch.bfloat16, 2), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I32": (torch.int32, 4), "I64": (torch.int64, 8),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
INDEX_NAME = "model.safetensors.index.json"


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

    def byte_range(self, name: str) -> Tuple[int, int, int]:
        """(file descriptor, offset in the file, bytes) of a tensor's data, for readers that
        bring the bytes into memory of their own."""
        _, _, b, e = self.entries[name]
        return self._f.fileno(), self._base + b, e - b

    def close(self):
        # tensors handed out keep the map alive through the buffer protocol
        self._f.close()


class SafetensorsFolder:
    """All tensors of a model folder: `model.safetensors`, or the shards an index names
    (`model.safetensors.index.json` -> `weight_map`: tensor name -> file)."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, INDEX_NAME)
        self.files: List[SafetensorsFile] = []
        self.where: Dict[str, SafetensorsFile] = {}
        weight_map: Optional[Dict[str, str]] = None
        if os.path.isfile(single):
            paths = [single]
        elif os.path.isfile(index):
            try:
                with open(index, "r", encoding="utf-8") as f:
                    weight_map = json.load(f).get("weight_map")
            except (OSError, json.JSONDecodeError, AttributeError) as e:
                raise WeightError(f"{index}: cannot read the index ({e})") from None
            if not isinstance(weight_map, dict) or not weight_map or \
                    not all(isinstance(k, str) and isinstance(v, str) for k, v in weight_map.items()):
                raise WeightError(f"{index}: 'weight_map' must map tensor names to file names")
            # a file of the index lies in the folder itself: no path that leads elsewhere is followed
            outside = sorted({v for v in weight_map.values()
                              if os.path.basename(v) != v or v in ("", ".", "..") or os.path.isabs(v)})
            if outside:
                raise WeightError(f"{index}: the index names files outside the model folder: {', '.join(outside)}")
            paths = [os.path.join(folder, v) for v in sorted(set(weight_map.values()))]
            absent = [os.path.basename(p) for p in paths if not os.path.isfile(p)]
            if absent:
                raise WeightError(f"{folder}: the index names files that are not there: {', '.join(absent)}")
        else:
            raise WeightError(f"{folder}: neither model.safetensors nor {INDEX_NAME}")
        for p in paths:
            sf = SafetensorsFile(p)
            self.files.append(sf)
            for n in sf.names():
                if n in self.where:
                    raise WeightError(f"{folder}: tensor {n} appears in two files "
                                      f"({os.path.basename(self.where[n].path)} and {os.path.basename(p)})")
                self.where[n] = sf
        if weight_map is not None:
            wrong = sorted(n for n, v in weight_map.items()
                           if n not in self.where or os.path.basename(self.where[n].path) != os.path.basename(v))
            if wrong:
                raise WeightError(f"{folder}: the index places tensors in files that do not hold them: {', '.join(wrong)}")

    def names(self) -> List[str]:
        return list(self.where)

    def info(self, name):
        return self.where[name].info(name)

    def tensor(self, name):
        return self.where[name].tensor(name)

    def byte_range(self, name):
        return self.where[name].byte_range(name)



class SafetensorsWriter:
    """Writes one file tensor by tensor: the header comes first, from the names, dtypes and
    shapes given up front; `write` then takes the tensors in that order and appends their
    bytes, so no more than one tensor is held at a time."""

    def __init__(self, path: str, layout: Sequence[Tuple[str, torch.dtype, Tuple[int, ...]]], metadata=None):
        header = {}
        if metadata:
            header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
        off = 0
        self._expect: List[Tuple[str, torch.dtype, Tuple[int, ...], int]] = []
        for name, dtype, shape in layout:
            if dtype not in _NAMES:
                raise WeightError(f"cannot store dtype {dtype} of {name}")
            if name in header:
                raise WeightError(f"{path}: tensor {name} is named twice")
            n = _DTYPES[_NAMES[dtype]][1]
            for s in shape:
                n *= int(s)
            header[name] = {"dtype": _NAMES[dtype], "shape": [int(s) for s in shape], "data_offsets": [off, off + n]}
            self._expect.append((name, dtype, tuple(int(s) for s in shape), n))
            off += n
        self.data_bytes = off
        hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
        hj += b" " * ((8 - len(hj) % 8) % 8)
        self.path = path
        self._f = open(path, "wb")
        self._f.write(struct.pack("<Q", len(hj)))
        self._f.write(hj)
        self._next = 0

    def write(self, name: str, t: torch.Tensor) -> None:
        if self._next >= len(self._expect):
            raise WeightError(f"{self.path}: tensor {name} is one more than the header names")
        want, dtype, shape, n = self._expect[self._next]
        if name != want or t.dtype != dtype or tuple(t.shape) != shape:
            raise WeightError(f"{self.path}: expected {want} {dtype} {list(shape)} next, "
                              f"got {name} {t.dtype} {list(t.shape)}")
        t = t.detach().cpu().contiguous()
        if n:
            self._f.write(memoryview(t.view(torch.uint8).reshape(-1).numpy()))
        self._next += 1

    def close(self) -> None:
        self._f.close()
        if self._next != len(self._expect):
            raise WeightError(f"{self.path}: {len(self._expect) - self._next} tensors of the header were never written")

    def __enter__(self):
        return self

    def __exit__(self, et, ev, tb):
        if et is None:
            self.close()
        else:
            self._f.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write tensors that are all at hand, in the given order."""
    items = [(n, t.detach()) for n, t in tensors]
    with SafetensorsWriter(path, [(n, t.dtype, tuple(t.shape)) for n, t in items], metadata) as w:
        for n, t in items:
            w.write(n, t)


def plan_shards(layout: Sequence[Tuple[str, torch.dtype, Tuple[int, ...]]], shard_bytes: Optional[int]) -> List[List[int]]:
    """Indices of `layout` per file: in order, a new file whenever the next tensor would
    take the current one beyond `shard_bytes` (None: one file)."""
    shards: List[List[int]] = [[]]
    used = 0
    for i, (name, dtype, shape) in enumerate(layout):
        n = _DTYPES[_NAMES[dtype]][1]
        for s in shape:
            n *= int(s)
        if shard_bytes and shards[-1] and used + n > shard_bytes:
            shards.append([])
            used = 0
        shards[-1].append(i)
        used += n
    return shards


def shard_file_name(i: int, n: int) -> str:
    return "model.safetensors" if n == 1 else f"model-{i + 1:05d}-of-{n:05d}.safetensors"


def write_index(folder: str, weight_map: Dict[str, str], total_size: int) -> None:
    with open(os.path.join(folder, INDEX_NAME), "w", encoding="utf-8") as f:
        json.dump({"metadata": {"total_size": int(total_size)}, "weight_map": weight_map}, f, indent=2)
