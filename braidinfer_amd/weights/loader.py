"""Weights by tensor name: what a model needs (`TensorSpec`), reading it from a folder
with one error for everything that does not fit, bringing it onto the GPU, and writing
a folder of seeded random weights.

The reference searches candidate names per tensor and takes the first that exists
(crates/braidinfer-runtime/src/weights.rs:273-288, model_load.rs:624-744), copies bf16
bytes verbatim (weights.rs:292-313) and asserts on a size mismatch (:301-307).  Here the
names are exact, and missing, unexpected and misshapen tensors are reported together.

Load mechanics.  The reference pins the mapped shards with `hipHostRegister` and copies
tensor by tensor with a synchronous `hipMemcpy` (model_load.rs:196-215); its other
format goes into one arena with a bulk copy (:316-364).  Here the parts of a model pull
their tensors from a *source* one at a time (`FolderTensors`, `RandomTensors`), build what
they keep (fused, interleaved, blocked matrices) inside one device allocation sized
beforehand (`WeightArena`), and drop what they pulled: the file's bytes go through two
pinned staging buffers (allocated pinned, never registered) with asynchronous copies on
a stream of their own, so reading the next piece overlaps the copy of the last, and host
memory stays at the staging buffers whatever the model's size.
"""
from __future__ import annotations

import json
import os
import time
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass, field
from typing import Dict, Iterable, Iterator, List, Optional, Sequence, Tuple

import torch

from ..errors import WeightError
from .random_weights import random_tensor, random_tensors
from .safetensors_io import (SafetensorsFolder, SafetensorsWriter, plan_shards, shard_file_name, write_index,
                             write_safetensors)


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part needs.  kind: "matrix" (follows the compute dtype unless stored in
    32-bit), "vector" (small float parameters, always widened to float32), "int" (integer
    table, kept as int32).  init: "normal" | "ones" | "zeros" for random weights."""

    name: str
    shape: Tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"


def _target_dtype(spec: TensorSpec, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if spec.kind == "int":
        return torch.int32
    if spec.kind == "vector":
        return torch.float32
    if stored == torch.float32:
        return torch.float32          # a tensor stored in 32-bit stays so
    return compute                    # bf16 stays bf16, or is widened for the 32-bit path


def _esize(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


ARENA_ALIGN = 256


def resident_bytes(specs: Sequence[TensorSpec], dtype_of) -> int:
    """Room for what the parts keep of these tensors: every tensor in its target dtype,
    rounded up to the arena's alignment, plus up to 15 rows of padding for a matrix that
    is kept in blocks of 16 rows."""
    total = 0
    for s in specs:
        e = _esize(dtype_of(s))
        n = _numel(s.shape) * e
        if len(s.shape) == 2:
            n += 15 * int(s.shape[1]) * e
        total += -(-n // ARENA_ALIGN) * ARENA_ALIGN + ARENA_ALIGN
    return total


class WeightArena:
    """One device allocation that the resident weights are carved from, in load order.
    What does not fit (a part that keeps more than its tensors' bytes) is allocated on its
    own and counted in `spilled`."""

    def __init__(self, device, nbytes: int):
        self.device = torch.device(device)
        self.buf = torch.empty(max(int(nbytes), ARENA_ALIGN), dtype=torch.uint8, device=self.device)
        self.used = 0
        self.spilled = 0

    def empty(self, shape, dtype: torch.dtype) -> torch.Tensor:
        n = _numel(shape) * _esize(dtype)
        start = -(-self.used // ARENA_ALIGN) * ARENA_ALIGN
        if start + n > self.buf.numel():
            self.spilled += n
            return torch.empty(tuple(shape), dtype=dtype, device=self.device)
        self.used = start + n
        return self.buf[start:start + n].view(dtype).view(tuple(int(s) for s in shape))

    def holds(self, t: torch.Tensor) -> bool:
        return t.untyped_storage().data_ptr() == self.buf.untyped_storage().data_ptr()


@dataclass
class LoadProfile:
    """Where the time of a load went."""

    tensors: int = 0
    file_bytes: int = 0
    read_seconds: float = 0.0        # host time in reads from the files into the staging buffers
    wait_seconds: float = 0.0        # host time waiting for a staging buffer's copy to end
    seconds: float = 0.0             # wall time of the whole load
    arena_bytes: int = 0
    arena_used: int = 0
    spilled_bytes: int = 0
    started: float = field(default_factory=time.perf_counter)

    def line(self) -> str:
        gbs = self.file_bytes / self.seconds / 1e9 if self.seconds > 0 else 0.0
        return (f"LOAD PROFILE: {self.tensors} tensors, {self.file_bytes / 1e9:.3f} GB in {self.seconds * 1e3:.0f} ms "
                f"= {gbs:.2f} GB/s (file reads {self.read_seconds * 1e3:.0f} ms, waits for copies "
                f"{self.wait_seconds * 1e3:.0f} ms), arena {self.arena_used / 1e9:.3f} of {self.arena_bytes / 1e9:.3f} GB"
                + (f", {self.spilled_bytes / 1e6:.1f} MB outside it" if self.spilled_bytes else ""))


def check_folder(folder: str, st: SafetensorsFolder, specs: Sequence[TensorSpec],
                 allow_unexpected: Sequence[str] = ()) -> None:
    """One `WeightError` that lists every missing, unexpected and misshapen tensor."""
    have = set(st.names())
    want = {s.name: s for s in specs}
    missing = sorted(n for n in want if n not in have)
    unexpected = sorted(n for n in have if n not in want and n not in allow_unexpected)
    mismatched = []
    for n, s in want.items():
        if n not in have:
            continue
        dt, shape = st.info(n)
        ok_dtype = (dt in (torch.int32, torch.int64)) if s.kind == "int" else (dt in (torch.bfloat16, torch.float32))
        if tuple(shape) != tuple(s.shape) or not ok_dtype:
            mismatched.append((n, tuple(s.shape), tuple(shape), str(dt).replace("torch.", "")))
    if missing or unexpected or mismatched:
        lines = [f"{folder}: the tensors do not match the model"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        for n, exp, got, dt in mismatched:
            lines.append(f"  wrong shape or dtype: {n}: expected {list(exp)}, found {list(got)} {dt}")
        raise WeightError("\n".join(lines), missing, unexpected, mismatched)


def _int32_checked(folder: str, name: str, t: torch.Tensor) -> torch.Tensor:
    if t.dtype == torch.int64 and t.numel() and (int(t.max()) > 2**31 - 1 or int(t.min()) < -2**31):
        raise WeightError(f"{folder}: integer table {name} does not fit in int32")
    return t.to(torch.int32)


class FolderTensors:
    """The tensors of a model folder as a read-only mapping name -> tensor on `device` in
    its target dtype.  Nothing is read before it is asked for, and nothing is kept: every
    `source[name]` brings the tensor from the file again.  Checked against `specs` when it
    is made.  On a GPU the bytes travel through pinned staging buffers (see the module's
    text); `profile` says how long that took."""

    def __init__(self, folder: str, specs: Sequence[TensorSpec], device, compute_dtype: torch.dtype,
                 allow_unexpected: Sequence[str] = (), staging_bytes: int = 64 << 20, read_threads: int = 4):
        self.folder = folder
        self.st = SafetensorsFolder(folder)
        check_folder(folder, self.st, specs, allow_unexpected)
        self.device = torch.device(device)
        self.compute_dtype = compute_dtype
        self.specs = {s.name: s for s in specs}
        self._have = set(self.st.names())
        self.profile = LoadProfile()
        self._staging_bytes = max(int(staging_bytes), 1 << 16)
        self._read_threads = max(1, int(read_threads))
        self._pinned: List[torch.Tensor] = []
        self._events: List[Optional[torch.cuda.Event]] = []
        self._turn = 0
        self._copy_stream = None
        self._pool: Optional[ThreadPoolExecutor] = None

    # -- mapping ---------------------------------------------------------------------
    def __contains__(self, name: str) -> bool:
        return name in self._have

    def names(self) -> List[str]:
        return list(self._have)

    def target_dtype(self, spec: TensorSpec) -> torch.dtype:
        return _target_dtype(spec, self.st.info(spec.name)[0], self.compute_dtype)

    def resident_bytes(self) -> int:
        return resident_bytes(list(self.specs.values()), self.target_dtype)

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._have:
            raise KeyError(name)
        spec = self.specs.get(name) or TensorSpec(name, tuple(self.st.info(name)[1]))
        stored, shape = self.st.info(name)
        target = _target_dtype(spec, stored, self.compute_dtype)
        self.profile.tensors += 1
        if self.device.type == "cpu" or spec.kind == "int" or _numel(shape) == 0:
            t = self.st.tensor(name)
            if spec.kind == "int":
                t = _int32_checked(self.folder, name, t)
            self.profile.file_bytes += t.numel() * t.element_size()
            return t.to(device=self.device, dtype=target, copy=True)
        raw = self._stream(name, stored, shape)
        if stored == target:
            return raw
        from .. import kernels as K
        out = torch.empty(tuple(shape), dtype=target, device=self.device)
        K.convert(raw, out)            # bfloat16 -> float32 (vectors, and matrices on the 32-bit path)
        return out

    # -- file -> pinned staging -> device ------------------------------------------------
    def _setup(self) -> None:
        if self._copy_stream is None:
            self._copy_stream = torch.cuda.Stream(device=self.device)
            self._pinned = [torch.empty(self._staging_bytes, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
            self._views = [memoryview(p.numpy()) for p in self._pinned]
            self._events = [None, None]
            if self._read_threads > 1:
                self._pool = ThreadPoolExecutor(self._read_threads)

    @staticmethod
    def _pread(fd: int, view: memoryview, offset: int) -> None:
        done = 0
        n = len(view)
        while done < n:
            got = os.preadv(fd, [view[done:]], offset + done)
            if got <= 0:
                raise WeightError("a model file ended before its tensors did (truncated while reading)")
            done += got

    def _read(self, fd: int, view: memoryview, offset: int) -> None:
        n = len(view)
        if self._pool is None or n < (8 << 20):
            self._pread(fd, view, offset)
            return
        k = self._read_threads
        piece = -(-n // k)
        piece = -(-piece // 4096) * 4096
        jobs = [self._pool.submit(self._pread, fd, view[a:min(n, a + piece)], offset + a) for a in range(0, n, piece)]
        for j in jobs:
            j.result()

    def _stream(self, name: str, stored: torch.dtype, shape) -> torch.Tensor:
        self._setup()
        fd, off, nbytes = self.st.byte_range(name)
        dst = torch.empty(tuple(shape), dtype=stored, device=self.device)
        flat = dst.view(-1).view(torch.uint8)
        cur = torch.cuda.current_stream(self.device)
        # the block under `dst` may have been freed a moment ago by work still queued on the
        # current stream: the copies start after that work
        self._copy_stream.wait_stream(cur)
        prof = self.profile
        for a in range(0, nbytes, self._staging_bytes):
            n = min(self._staging_bytes, nbytes - a)
            k = self._turn
            self._turn ^= 1
            ev = self._events[k]
            if ev is not None:
                t0 = time.perf_counter()
                ev.synchronize()
                prof.wait_seconds += time.perf_counter() - t0
            t0 = time.perf_counter()
            self._read(fd, self._views[k][:n], off + a)
            prof.read_seconds += time.perf_counter() - t0
            with torch.cuda.stream(self._copy_stream):
                flat[a:a + n].copy_(self._pinned[k][:n], non_blocking=True)
                if ev is None:
                    ev = self._events[k] = torch.cuda.Event()
                ev.record(self._copy_stream)
        cur.wait_stream(self._copy_stream)
        prof.file_bytes += nbytes
        return dst

    def finish(self, arena: Optional[WeightArena] = None) -> LoadProfile:
        """Wait for the last copies, give the staging buffers back, close the books."""
        if self._copy_stream is not None:
            self._copy_stream.synchronize()
            torch.cuda.current_stream(self.device).synchronize()
        if self._pool is not None:
            self._pool.shutdown()
            self._pool = None
        self._views = []
        self._pinned = []
        self._events = []
        p = self.profile
        p.seconds = time.perf_counter() - p.started
        if arena is not None:
            p.arena_bytes, p.arena_used, p.spilled_bytes = arena.buf.numel(), arena.used, arena.spilled
        return p


class RandomTensors:
    """Seeded random weights as a source: `source[name]` is made on `device` when asked for,
    bfloat16 values (the same bits a random-weights folder of that seed holds), widened
    to float32 for vectors and for the 32-bit path."""

    def __init__(self, specs: Sequence[TensorSpec], seed: int, device, compute_dtype: torch.dtype, std: float = 0.02,
                 vector_jitter: float = 0.0):
        self.specs = {s.name: (i, s) for i, s in enumerate(specs)}
        self.seed, self.device, self.compute_dtype = int(seed), torch.device(device), compute_dtype
        self.std, self.vector_jitter = float(std), float(vector_jitter)
        self.profile = LoadProfile()

    def __contains__(self, name: str) -> bool:
        return name in self.specs

    def names(self) -> List[str]:
        return list(self.specs)

    def target_dtype(self, spec: TensorSpec) -> torch.dtype:
        return _target_dtype(spec, torch.bfloat16, self.compute_dtype)

    def resident_bytes(self) -> int:
        return resident_bytes([s for _, s in self.specs.values()], self.target_dtype)

    def __getitem__(self, name: str) -> torch.Tensor:
        i, spec = self.specs[name]
        t = random_tensor(spec, i, self.seed, self.device, torch.bfloat16, self.std, self.vector_jitter)
        self.profile.tensors += 1
        target = self.target_dtype(spec)
        if t.dtype == target:
            return t
        if self.device.type == "cpu":
            return t.to(target)
        from .. import kernels as K
        out = torch.empty(spec.shape, dtype=target, device=self.device)
        K.convert(t, out)
        return out

    def finish(self, arena: Optional[WeightArena] = None) -> LoadProfile:
        p = self.profile
        if self.device.type != "cpu":
            torch.cuda.current_stream(self.device).synchronize()
        p.seconds = time.perf_counter() - p.started
        if arena is not None:
            p.arena_bytes, p.arena_used, p.spilled_bytes = arena.buf.numel(), arena.used, arena.spilled
        return p


def load_tensors(folder: str, specs: Sequence[TensorSpec], device, compute_dtype: torch.dtype,
                 allow_unexpected: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """Exactly the tensors `specs` names, from `folder`, all at once as a dict (small models,
    tools, the CPU; a model on the GPU pulls from `FolderTensors` instead)."""
    src = FolderTensors(folder, specs, device, compute_dtype, allow_unexpected)
    out = {s.name: src[s.name] for s in specs}
    src.finish()
    return out


def write_model_folder(folder: str, config, specs: Sequence[TensorSpec], seed: int, std: float = 0.02,
                       vector_jitter: float = 0.0, dtype=torch.bfloat16, device="cpu",
                       shard_bytes: Optional[int] = None) -> str:
    """Random-weights mode: config.json and model.safetensors from a configuration and a
    seed.  Tensors are made one at a time (on `device`: a GPU makes a 7B-sized folder in
    the time it takes to write it) and appended to the file, whose header is written first
    from the shapes.  `shard_bytes` cuts the folder into files of about that size with a
    `model.safetensors.index.json`, as large checkpoints are shipped."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=2)
    layout = [(s.name, torch.int32 if s.kind == "int" else dtype, tuple(s.shape)) for s in specs]
    shards = plan_shards(layout, shard_bytes)
    weight_map: Dict[str, str] = {}
    total = 0
    for k, members in enumerate(shards):
        fname = shard_file_name(k, len(shards))
        with SafetensorsWriter(os.path.join(folder, fname), [layout[i] for i in members],
                               metadata={"format": "pt", "seed": seed}) as w:
            for i in members:
                w.write(specs[i].name, random_tensor(specs[i], i, seed, device, dtype, std, vector_jitter))
                weight_map[specs[i].name] = fname
            total += w.data_bytes
    if len(shards) > 1:
        write_index(folder, weight_map, total)
    return folder
