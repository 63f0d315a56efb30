"""Seeded random weights from this library's own counter-based generator.

A value is a pure function of (seed, index of the tensor in the model's name table,
element index), computed with 64-bit integer arithmetic and one float multiplication, so
the device kernel (`csrc/random_weights.hip`), the NumPy form below and any other
implementation of the same few lines give the same bits:

    mix(z):   z ^= z >> 30; z *= 0xBF58476D1CE4E5B9; z ^= z >> 27; z *= 0x94D049BB133111EB; z ^= z >> 31
    key     = mix(mix(seed + G) + (tensor + 1) * G)           G = 0x9E3779B97F4A7C15, all modulo 2^64
    word(c) = mix(key + (c + 1) * G)
    normal, element i:  s = the twelve 16-bit fields of word(3i), word(3i+1), word(3i+2) added up;
                        value = float32(s - 393210) * (float32(std) * 2^-16)
    one with jitter, element i:  u = float32(word(i) >> 40) * 2^-24;  value = 1 + (2u - 1) * jitter

Matrices are N(0, std) to the accuracy of a sum of twelve uniform numbers (exact mean and
variance, tails cut at 6 std); float32 values are the master, bfloat16 is their rounding
to nearest even (the reference's own rounding, crates/braidinfer-runtime/src/quant.rs:203-207).
Norm weights are exactly 1 unless a test asks for jitter.  The reference has no random
weights.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Iterable, Iterator, Optional, Sequence, Tuple

import numpy as np
import torch

_M = (1 << 64) - 1
_G = 0x9E3779B97F4A7C15
_CENTRE = 393210          # 12 * 65535 / 2


def _mix_int(z: int) -> int:
    z &= _M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
    return z ^ (z >> 31)


def tensor_key(seed: int, tensor_index: int) -> int:
    return _mix_int(_mix_int((int(seed) + _G) & _M) + ((int(tensor_index) + 1) * _G & _M))


def _mix(z: np.ndarray) -> np.ndarray:
    z = z ^ (z >> np.uint64(30))
    z = z * np.uint64(0xBF58476D1CE4E5B9)
    z = z ^ (z >> np.uint64(27))
    z = z * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _words(key: int, counters: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return _mix(np.uint64(key) + (counters + np.uint64(1)) * np.uint64(_G))


def _fields(w: np.ndarray) -> np.ndarray:
    m = np.uint64(0xFFFF)
    return ((w & m) + ((w >> np.uint64(16)) & m) + ((w >> np.uint64(32)) & m) + (w >> np.uint64(48))).astype(np.int64)


def normal_f32(key: int, n: int, std: float, first: int = 0) -> np.ndarray:
    """Elements first .. first + n - 1 of the normal tensor with this key, float32."""
    scale = np.float32(np.float32(std) * np.float32(2.0 ** -16))
    out = np.empty(n, dtype=np.float32)
    step = 1 << 20
    for a in range(0, n, step):
        b = min(n, a + step)
        i = np.arange(first + a, first + b, dtype=np.uint64)
        with np.errstate(over="ignore"):
            c = i * np.uint64(3)
            s = _fields(_words(key, c)) + _fields(_words(key, c + np.uint64(1))) + _fields(_words(key, c + np.uint64(2)))
        out[a:b] = (s - _CENTRE).astype(np.float32) * scale
    return out


def ones_f32(key: int, n: int, jitter: float, first: int = 0) -> np.ndarray:
    if not jitter:
        return np.ones(n, dtype=np.float32)
    i = np.arange(first, first + n, dtype=np.uint64)
    u = (_words(key, i) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    d = ((u + u) - np.float32(1.0)) * np.float32(jitter)
    return (np.float32(1.0) + d).astype(np.float32)


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round to nearest even, as quant.rs:203-207 (finite values only)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return ((u + (((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF))) >> np.uint32(16)).astype(np.uint16)


def _cpu_tensor(spec, key: int, dtype: torch.dtype, std: float, jitter: float) -> torch.Tensor:
    n = 1
    for s in spec.shape:
        n *= int(s)
    vals = ones_f32(key, n, jitter) if spec.init == "ones" else normal_f32(key, n, std)
    if dtype == torch.bfloat16:
        return torch.from_numpy(f32_to_bf16_bits(vals).view(np.int16)).view(torch.bfloat16).reshape(spec.shape)
    return torch.from_numpy(vals).reshape(spec.shape)


def random_tensor(spec, tensor_index: int, seed: int, device="cpu", dtype=torch.bfloat16, std: float = 0.02,
                  vector_jitter: float = 0.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The tensor `spec` names, as entry `tensor_index` of its model's name table: integer
    tables and "zeros" are zero, "ones" are 1 (plus jitter), everything else is normal.
    On a GPU the values are made there by the kernel; on the CPU by NumPy: the same bits."""
    device = torch.device(device)
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    key = tensor_key(seed, tensor_index)
    if device.type == "cpu":
        t = _cpu_tensor(spec, key, dtype, std, vector_jitter)
        if out is not None:
            out.copy_(t)
            return out
        return t
    from .. import kernels as K
    t = out if out is not None else torch.empty(spec.shape, dtype=dtype, device=device)
    if spec.init == "ones":
        K.random_ones(t, key, float(vector_jitter))
    else:
        K.random_normal(t, key, float(std))
    return t


def random_tensors(specs: Sequence, seed: int, device="cpu", dtype=torch.bfloat16, std: float = 0.02,
                   vector_jitter: float = 0.0) -> Iterator[Tuple[str, torch.Tensor]]:
    """(name, tensor) in the order of the name table `specs`."""
    for i, s in enumerate(specs):
        yield s.name, random_tensor(s, i, seed, device, dtype, std, vector_jitter)
