"""Compiles the HIP sources beside this file for gfx950 and loads them with ctypes.

Each source file becomes one shared library (`br_<name>.so`), built on first use and
reused while its sources and flags are unchanged, so a run compiles only what its model
and dtype need.  Libraries are written beside the sources when that folder is writable,
else under ``$BRAIDINFER_BUILD_DIR`` or a per-user folder in the temporary directory.
A compile prints a line when it starts, every few seconds while it runs, and when it
ends, on standard error.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Iterable, List, Optional

from ..errors import KernelError

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from float code on this target.
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-inline-asm"]
MODULES: Dict[str, List[str]] = {
    "elementwise": ["elementwise.hip"],
    "gemm_f32": ["gemm_f32.hip"],
    "attention_simple": ["attention_simple.hip"],
    "sampling": ["sampling.hip"],
    "gemm_bf16": ["gemm_bf16.hip"],
    "attention_bf16": ["attention_bf16.hip"],
    "random_weights": ["random_weights.hip"],
}
HEADERS = ["common.h", "no_alloc.h"]

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def _log(msg: str) -> None:
    print(f"[braidinfer_amd build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _digest(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for f in MODULES[name] + HEADERS:
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(f.encode())
            h.update(fh.read())
    return h.hexdigest()


def _build_dirs() -> List[str]:
    dirs = []
    env = os.environ.get("BRAIDINFER_BUILD_DIR")
    if env:
        dirs.append(env)
    dirs.append(HERE)
    dirs.append(os.path.join(tempfile.gettempdir(), f"braidinfer_amd_{os.getuid()}"))
    return dirs


def _file_digest(path: str) -> str:
    h = hashlib.sha256()
    with open(path, "rb") as f:
        for chunk in iter(lambda: f.read(1 << 20), b""):
            h.update(chunk)
    return h.hexdigest()


def _find_built(name: str, digest: str) -> Optional[str]:
    """A library counts as built when its tag names both the sources it was made from and
    the library file itself (a tag restored or copied without its library does not)."""
    for d in _build_dirs():
        so = os.path.join(d, f"br_{name}.so")
        tag = so + ".tag"
        if os.path.isfile(so) and os.path.isfile(tag):
            try:
                with open(tag) as f:
                    parts = f.read().split()
                if len(parts) == 2 and parts[0] == digest and parts[1] == _file_digest(so):
                    return so
            except OSError:
                pass
    return None


def _writable_dir() -> str:
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            fd, probe = tempfile.mkstemp(prefix=".probe_", dir=d)
            os.close(fd)
            os.unlink(probe)
            return d
        except OSError:
            continue
    raise KernelError("no writable folder to build the HIP kernels in; set BRAIDINFER_BUILD_DIR")


def compile_module(name: str, force: bool = False) -> str:
    """Build one module if it is not built for the current sources; return the path."""
    if name not in MODULES:
        raise KernelError(f"unknown kernel module {name!r}; known: {sorted(MODULES)}")
    for f in MODULES[name]:
        if not os.path.isfile(os.path.join(HERE, f)):
            raise KernelError(f"kernel source {f} is missing from {HERE}")
    digest = _digest(name)
    if not force:
        so = _find_built(name, digest)
        if so:
            return so
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelError(
            f"kernel module {name!r} is not built and hipcc was not found; this library has no "
            "fallback path (build with `python -c 'import __graft_entry__ as g; g.build()'`)")
    out_dir = _writable_dir()
    so = os.path.join(out_dir, f"br_{name}.so")
    tmp = so + f".tmp{os.getpid()}"
    cmd = [hipcc] + FLAGS + [os.path.join(HERE, f) for f in MODULES[name]] + ["-o", tmp]
    _log(f"compiling {name} for {ARCH} ...")
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=out_dir)
    out_chunks: List[bytes] = []
    reader = threading.Thread(target=lambda: out_chunks.append(proc.stdout.read()), daemon=True)
    reader.start()
    last = t0
    while proc.poll() is None:
        time.sleep(0.2)
        if time.time() - last > 10:
            last = time.time()
            _log(f"  still compiling {name} ({last - t0:.0f} s)")
    reader.join()
    text = b"".join(out_chunks).decode(errors="replace")
    text = "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise KernelError(f"hipcc failed for {name} (exit {proc.returncode}):\n{text}")
    os.replace(tmp, so)
    with open(so + ".tag", "w") as f:
        f.write(f"{digest} {_file_digest(so)}\n")
    _log(f"built {name} in {time.time() - t0:.1f} s -> {so}")
    return so


def build_all(force: bool = True, names: Optional[Iterable[str]] = None, jobs: int = 4) -> List[str]:
    """Compile every module, by default also those already built for the current sources."""
    names = [n for n in (names or MODULES) if all(os.path.isfile(os.path.join(HERE, f)) for f in MODULES[n])]
    results: Dict[str, str] = {}
    errors: List[str] = []
    sem = threading.Semaphore(jobs)

    def work(n):
        with sem:
            try:
                results[n] = compile_module(n, force=force)
            except KernelError as e:
                errors.append(str(e))

    threads = [threading.Thread(target=work, args=(n,)) for n in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise KernelError("\n".join(errors))
    return [results[n] for n in names]


def load(name: str) -> ctypes.CDLL:
    """The module's library, compiled first if needed.  torch must already be imported
    so that the library binds to the HIP runtime torch has loaded."""
    with _lock:
        lib = _loaded.get(name)
        if lib is None:
            import torch  # noqa: F401  (loads libamdhip64 before our library asks for it)
            so = compile_module(name)
            try:
                lib = ctypes.CDLL(so)
            except OSError as e:
                raise KernelError(f"cannot load {so}: {e}") from None
            _loaded[name] = lib
        return lib


def loaded_modules() -> List[str]:
    return sorted(_loaded)
