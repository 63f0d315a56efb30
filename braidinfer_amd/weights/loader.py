"""Weights by tensor name: what a model needs (`TensorSpec`), reading it from a folder
with one error for everything that does not fit, and seeded random weights.

The reference searches candidate names per tensor and takes the first that exists
(crates/braidinfer-runtime/src/weights.rs:273-288, model_load.rs:624-744), copies bf16
bytes verbatim (weights.rs:292-313) and asserts on a size mismatch (:301-307).  Here the
names are exact, and missing, unexpected and misshapen tensors are reported together.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from ..errors import WeightError
from .safetensors_io import SafetensorsFolder, write_safetensors


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


def load_tensors(folder: str, specs: Sequence[TensorSpec], device, compute_dtype: torch.dtype,
                 allow_unexpected: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """Read exactly the tensors `specs` names from `folder` onto `device`."""
    st = SafetensorsFolder(folder)
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
    out: Dict[str, torch.Tensor] = {}
    for s in specs:
        t = st.tensor(s.name)
        if s.kind == "int" and t.dtype == torch.int64:
            if t.numel() and (int(t.max()) > 2**31 - 1 or int(t.min()) < -2**31):
                raise WeightError(f"{folder}: integer table {s.name} does not fit in int32")
        out[s.name] = t.to(device=device, dtype=_target_dtype(s, t.dtype, compute_dtype), copy=True)
    return out


def random_tensors(specs: Sequence[TensorSpec], seed: int, device="cpu", dtype=torch.bfloat16,
                   std: float = 0.02, vector_jitter: float = 0.0) -> Iterable[Tuple[str, torch.Tensor]]:
    """Seeded weights in spec order: N(0, std) matrices, norm weights 1 (plus a uniform
    jitter of +-`vector_jitter` so tests can see a norm weight that is not applied)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    for s in specs:
        if s.kind == "int":
            yield s.name, torch.zeros(s.shape, dtype=torch.int32, device=device)
        elif s.init == "ones":
            t = torch.ones(s.shape, dtype=torch.float32, device=device)
            if vector_jitter:
                t += (torch.rand(s.shape, generator=gen, device=device) * 2 - 1) * vector_jitter
            yield s.name, t.to(dtype)
        elif s.init == "zeros":
            yield s.name, torch.zeros(s.shape, dtype=dtype, device=device)
        else:
            # generated in float32 in chunks so that a 7B-sized matrix never needs a
            # float32 copy of itself
            t = torch.empty(s.shape, dtype=dtype, device=device)
            flat = t.view(-1)
            step = 1 << 24
            for i in range(0, flat.numel(), step):
                n = min(step, flat.numel() - i)
                flat[i:i + n] = (torch.randn(n, generator=gen, device=device, dtype=torch.float32) * std).to(dtype)
            yield s.name, t


def write_model_folder(folder: str, config, specs: Sequence[TensorSpec], seed: int, std: float = 0.02,
                       vector_jitter: float = 0.0, dtype=torch.bfloat16) -> str:
    """Random-weights mode: config.json and model.safetensors from a configuration and a seed."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(specs, seed, "cpu", dtype, std, vector_jitter),
                      metadata={"format": "pt", "seed": seed})
    return folder
